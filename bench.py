#!/usr/bin/env python3
"""Benchmark of the seblas conv/GEMM hot path on one MI355X.

Default workload (benchmark configuration 2): the convolution layers of ResNet-56 on CIFAR-shaped tensors, fp32 NCHW,
batch 128. One *step* = forward + data-gradient + weight-gradient of every 3x3 conv layer of the network's three
stages and two stride-2 transitions, with the layer multiplicities of the reference's archived model
(archive/Resnet56: 19x 16->16@32, 17x 32->32@16, 18x 64->64@8, 1x 16->32 s2, 1x 32->64 s2), on synthetic
N(0,1) activations/gradients and He-normal filters already resident in HBM. Flops are nominal
(2*N*OC*OH*OW*IC*FH*FW per pass; zeros from stride/padding are not discounted).

The timed step issues, per layer, crb_conv_fwd and crb_conv_bwd_sliced (both gradients in one launch) and sums all
weight-gradient slices with one crb_sum_slices_multi at its end. `three_call_step` times the same work through the
reference's own call sequence (conv, convDerive, convError as three separate calls per layer: crb_conv_fwd,
crb_conv_dgrad, crb_conv_wgrad; seann/operands/seblas/Conv2D.cu:8-29), also over exactly K steps.

Cache state: a layer shape is run `mult` times on ONE set of X / W / dY buffers, so a launch finds its inputs in L2 or
the memory-side cache (in a whole network, where inputs arrive from the previous operator, the same kernels measure 4-8 %
longer). `extra.cold_ms_per_step` repeats both step forms with every layer instance on buffers of its own (about 1 GB of
distinct operands per step, beyond L2 and the 256 MB memory-side cache).

Prints ONE JSON line. `value` is TFLOP/s over the timed steps; `extra` carries images/s and the 4096^3 sgemm rate.
`roofline` describes the kernel that takes the most time in the step, timed per launch with HIP events on the
launch stream in a separate instrumented pass. `cpu_baseline` is the CPU oracle on a bounded sample.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--report FILE]   (--report adds every benchmark configuration)
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3  # 256 CU x 2.4 GHz x 256 flop/clk/CU
PEAK_HBM_GBS = 8000.0

# (name, IC, H, OC, stride, multiplicity) — 3x3, pad 1
RESNET56 = [
    ("L1_16-16@32", 16, 32, 16, 1, 19),
    ("L2_32-32@16", 32, 16, 32, 1, 17),
    ("L3_64-64@8", 64, 8, 64, 1, 18),
    ("T1_16-32s2", 16, 32, 32, 2, 1),
    ("T2_32-64s2", 32, 16, 64, 2, 1),
]
BATCH = 128


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--report", type=str, default=None, help="also time every benchmark configuration and write a JSON report")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the `configs` block (one figure per other benchmark configuration; a few seconds of GPU time)")
    ap.add_argument("--traffic", nargs="?", const="resnet56", default=None, choices=("resnet56", "densenet"),
                    help="only run every (layer, pass) call of the workload (default) or of the DenseNet-BC-100 shapes of the "
                         "report three times, each group behind a one-float fill launch as a separator, and print the order: "
                         "under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE the dispatch list then splits into calls "
                         "(profiles/resnet56_conv_step_b128.md and profiles/densenet_bc100_hbm_bytes_per_call.md are built from it)")
    ap.add_argument("--calibrate", action="store_true",
                    help="only run a plain streaming kernel of known size (a += b on 64 Mi floats: reads 512 MiB, writes "
                         "256 MiB per launch) so hardware byte counters can be scaled against it, then exit")
    return ap.parse_args()


class Layer:
    def __init__(self, torch, capi, dev, name, IC, H, OC, s, mult, seed, batch=BATCH, F=3, pad=1, bias=False, device_rng=False):
        self.name, self.mult = name, mult
        self.g = capi.ConvGeom.make(batch, IC, H, H, OC, F, F, s, s, pad, pad)
        g = self.g
        # device_rng: values drawn on the GPU (timing-only layers: many tensors, nothing compared with a CPU result)
        gen = torch.Generator(device=dev if device_rng else "cpu").manual_seed(seed)

        def randn(*shape):
            return torch.randn(*shape, generator=gen, device=dev) if device_rng else torch.randn(*shape, generator=gen).to(dev)

        self.X = randn(batch, IC, H, H)
        self.W = randn(OC, IC, F, F) * math.sqrt(2.0 / (IC * F * F))
        self.dY = randn(batch, OC, g.OH, g.OW)
        self.b = randn(OC) if bias else None
        self.Y = torch.empty(batch, OC, g.OH, g.OW, device=dev)
        self.dX = torch.empty(batch, IC, H, H, device=dev)
        self.dW = torch.zeros(OC, IC, F, F, device=dev)
        nbytes = capi.conv_wgrad_workspace_bytes(g)
        self.ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=dev) if nbytes else None
        # The timed step runs a layer shape `mult` times, as the network has `mult` such layers; with the slice summation
        # postponed to the end of the backward pass every one of them owns its slices and its dW until then.
        self.n_slices = capi.conv_bwd_slices(g)
        self.ws_each = [torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=dev) for _ in range(mult)] if self.n_slices else []
        self.dW_each = [torch.zeros(OC, IC, F, F, device=dev) for _ in range(mult)] if self.n_slices else []
        self.flops = 2.0 * batch * OC * g.OH * g.OW * IC * F * F
        nb = 0 if self.b is None else OC
        self.bytes = {
            "fwd": 4.0 * (self.X.numel() + self.W.numel() + self.Y.numel() + nb),
            "dgrad": 4.0 * (self.dY.numel() + self.W.numel() + self.dX.numel()),
            "wgrad": 4.0 * (self.dY.numel() + self.X.numel() + 2 * self.dW.numel()),
        }
        # both gradients in one call: dY is read by both halves but counted once
        self.bytes["bwd"] = 4.0 * (self.dY.numel() + self.W.numel() + self.dX.numel() + self.X.numel() + 2 * self.dW.numel())
        self.bytes["bwd_sliced"] = self.bytes["bwd"]  # its share of the final summation included
        self.capi = capi
        self.sets = None
        self._prepare()

    def make_cold_sets(self, torch, dev):
        """One X / dY / Y / dX set per layer instance (the filters and their gradients are per instance already)."""
        self.sets = [(torch.randn_like(self.X), torch.randn_like(self.dY), torch.empty_like(self.Y), torch.empty_like(self.dX),
                      self.W.clone(), torch.zeros_like(self.dW)) for _ in range(self.mult)]

    def fwd_cold(self, k):
        X, dY, Y, dX, W, dW = self.sets[k]
        self.capi.conv_fwd(W, X, Y, self.b, self.g)

    def bwd_sliced_cold(self, k):
        X, dY, Y, dX, W, dW = self.sets[k]
        self.capi.conv_bwd_sliced(W, dY, X, dX, self.g, self.ws_each[k])

    def bwd_cold(self, k):
        X, dY, Y, dX, W, dW = self.sets[k]
        self.capi.conv_bwd(W, dY, X, dX, dW, self.g, workspace=self.ws)

    def dgrad_wgrad_cold(self, k):
        X, dY, Y, dX, W, dW = self.sets[k]
        self.capi.conv_dgrad(W, dY, dX, self.g)
        self.capi.conv_wgrad(dY, X, dW, self.g, workspace=self.ws)

    # The per-call timing loops issue prepared calls (arguments converted once): through the plain ctypes wrappers a loop
    # is bound by 3.5-4.5 us of argument conversion per call, more than the small layers' kernels take.
    def _prepare(self):
        c, ws = self.capi, self.ws
        nbytes = 0 if ws is None else ws.numel() * ws.element_size()
        self._fwd = c.prepared("crb_conv_fwd", self.W, self.X, self.Y, self.b, self.g, 0, None)
        self._dgrad = c.prepared("crb_conv_dgrad", self.W, self.dY, self.dX, self.g, None)
        self._wgrad = c.prepared("crb_conv_wgrad", self.dY, self.X, self.dW, self.g, ws, nbytes, None)
        self._bwd = c.prepared("crb_conv_bwd", self.W, self.dY, self.X, self.dX, self.dW, self.g, ws, nbytes, None)
        self._bwd_sliced = [c.prepared("crb_conv_bwd_sliced", self.W, self.dY, self.X, self.dX, self.g, w, w.numel() * w.element_size(), None)
                            for w in self.ws_each]

    def fwd(self):
        self._fwd()

    def dgrad(self):
        self._dgrad()

    def wgrad(self):
        self._wgrad()

    def bwd(self):
        self._bwd()

    def bwd_sliced(self, k=0):
        self._bwd_sliced[k]()

    def slice_entries(self):
        return [(ws, dW, self.n_slices) for ws, dW in zip(self.ws_each, self.dW_each)]

    def passes(self):
        """(name, call, flops, part of the timed step). The step runs fwd and bwd_sliced per layer and one summation of all
        slices at its end; the self-contained backward call and the two gradients alone are listed too."""
        out = [("fwd", self.fwd, self.flops, True)]
        if self.n_slices:
            out.append(("bwd_sliced", self.bwd_sliced, 2 * self.flops, True))
        out += [("bwd", self.bwd, 2 * self.flops, not self.n_slices), ("dgrad", self.dgrad, self.flops, False),
                ("wgrad", self.wgrad, self.flops, False)]
        return out


# HBM bytes one call moves (read + written, all kernels of the call) come from the hardware counters FETCH_SIZE and
# WRITE_SIZE of `bench.py --traffic` under rocprofv3 --pmc, scaled by what the same counters read for a copy kernel of
# known size (`--calibrate`). They are a property of the kernels' access pattern, not of a run, so they are not measured
# here: the table "HBM bytes per call" of the tracked profile summary below is the one source, together with the commit
# and kernel names it was taken at.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "resnet56_conv_step_b128.md")


def measured_hbm_bytes():
    """{call key: bytes per call}, the commit the counters were taken at and the hash of the kernel sources they were taken
    on, from the tracked profile summary ({} if absent)."""
    table, commit, src_hash = {}, None, None
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
    except OSError:
        return table, commit, src_hash
    on = False
    for ln in lines:
        if ln.startswith("Counters taken at commit"):
            commit = ln.split("`")[1] if "`" in ln else None
        if ln.startswith("Kernel source hash"):
            src_hash = ln.split("`")[-2] if ln.count("`") >= 2 else None  # the line's last quoted token
        if ln.startswith("## HBM bytes per call"):
            on = True
            continue
        if on and ln.startswith("## "):
            break
        if on and ln.startswith("| ") and not ln.startswith("| call") and not ln.startswith("|---"):
            cells = [c.strip() for c in ln.strip("|").split("|")]
            try:
                table[cells[0].strip("`")] = float(cells[-1]) * 1e6  # last column: total MB per call
            except (ValueError, IndexError):
                pass
    return table, commit, src_hash


def device_clock_khz():
    """Peak engine clock of device 0 in kHz (hipDeviceAttributeClockRate), 0 if the runtime cannot be asked."""
    import ctypes

    try:
        hip = ctypes.CDLL("libamdhip64.so")
        v = ctypes.c_int(0)
        if hip.hipDeviceGetAttribute(ctypes.byref(v), 5, 0) == 0:  # 5 = hipDeviceAttributeClockRate
            return v.value
    except OSError:
        pass
    return 0


def event_time_ms(torch, fn, reps, warm=3):
    """Average duration of `fn` (ms) over `reps` back-to-back launches between two events on the launch stream."""
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / reps


def cpu_baseline(layers_spec, min_seconds=10.0):
    """CPU oracle on the same workload: whole ResNet-56 conv steps at the real batch, repeated until `min_seconds` of
    CPU work have been timed (at least one step), all host cores capped at 16."""
    import numpy as np

    from oracle import seblas_oracle as orc

    threads = min(os.cpu_count() or 1, 16)
    nb = BATCH
    rng = np.random.default_rng(0)
    work = []
    flops = 0.0
    for (_, IC, H, OC, s, mult) in layers_spec:
        OH = (H + 2 - 3) // s + 1
        X = rng.standard_normal((nb, IC, H, H)).astype(np.float32)
        W = (rng.standard_normal((OC, IC, 3, 3)) * math.sqrt(2.0 / (IC * 9))).astype(np.float32)
        dY = rng.standard_normal((nb, OC, OH, OH)).astype(np.float32)
        work.append((X, W, dY, np.zeros_like(W), H, s, mult))
        flops += 3 * mult * 2.0 * nb * OC * OH * OH * IC * 9
    steps, dt = 0, 0.0
    t0 = time.perf_counter()
    while steps == 0 or dt < min_seconds:
        for (X, W, dY, dW, H, s, mult) in work:
            for _ in range(mult):
                orc.conv(W, X, None, s, s, 1, 1, threads=threads)
                orc.convDerive(W, dY, (H, H), s, s, 1, 1, threads=threads)
                orc.convError(dY, X, dW, s, s, 1, 1, threads=threads)
        steps += 1
        dt = time.perf_counter() - t0
    return {
        "value": flops * steps / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "images_per_s": nb * steps / dt, "seconds": dt,
        "sample": f"{steps} full ResNet-56 conv steps (fwd+dgrad+wgrad, all 56 layers) at batch {nb}, "
                  f"fp32 loop oracle, {threads} threads",
    }


def full_network_steps():
    """The whole ResNet-56 / VGG-16 training steps (every operator, optimizer included) through the C++ seann host layer,
    each run by its own example program as a child process BEFORE this process touches the GPU. Returns {} when the
    programs are not built, when a profiler has already initialised the GPU in this process, or on any failure: the
    figures are an extra, the benchmark does not depend on them."""
    import subprocess

    if any(k.startswith(("ROCPROF", "ROCP_", "ROCTRACER")) for k in os.environ):
        return {}
    out = {}
    bindir = os.path.join(ROOT, "crusaderbackend_amd", "host", "examples", "bin")
    for key, exe, argv in (("resnet56_full_step", "resnet56_step", ["128", "10"]), ("vgg16_full_step_cpp", "vgg16_step", ["128", "10"])):
        path = os.path.join(bindir, exe)
        if not os.path.exists(path):
            continue
        try:
            r = subprocess.run([path] + argv, capture_output=True, text=True, timeout=120)
            if r.returncode == 0:
                out[key] = json.loads(r.stdout.strip().splitlines()[-1])
        except (OSError, subprocess.SubprocessError, ValueError, IndexError):
            pass
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build targets one GPU per process and has no multi-GPU path; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    full_net = {} if args.calibrate else full_network_steps()
    import torch

    from crusaderbackend_amd import capi

    capi.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)

    if args.calibrate:
        n = 64 << 20
        x, y = torch.ones(n, device=dev), torch.ones(n, device=dev)
        for _ in range(3):
            capi.tensor_add_inplace(x, y, n)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate": "add_inplace_kernel", "floats": n, "read_bytes": 8 * n, "write_bytes": 4 * n}))
        return

    if args.traffic == "densenet":
        # benchmark configuration 4: first / middle / last bottleneck of each stage and the stage's 3x3 layer, batch 64
        layers = []
        for (H, base) in ((32, 24), (16, 108), (8, 150)):
            for i in (0, 8, 15):
                layers.append(Layer(torch, capi, dev, f"1x1_{base + 12 * i}-48@{H}", base + 12 * i, H, 48, 1, 1, seed=300 + i, batch=64, F=1,
                                    pad=0, bias=True, device_rng=True))
            layers.append(Layer(torch, capi, dev, f"3x3_48-12@{H}", 48, H, 12, 1, 1, seed=400, batch=64, F=3, pad=1, bias=True, device_rng=True))
    else:
        layers = [Layer(torch, capi, dev, n, IC, H, OC, s, m, seed=10 + i) for i, (n, IC, H, OC, s, m) in enumerate(RESNET56)]
    if args.traffic:
        sep = torch.zeros(1, device=dev)
        order = []
        for L in layers:
            for pname, fn, _, _ in L.passes():
                if args.traffic == "densenet" and pname not in ("fwd", "dgrad", "wgrad"):
                    continue
                for _ in range(2):  # untimed: lets every kernel of the call load its code and grow nothing later
                    fn()
                torch.cuda.synchronize()
                capi.tensor_fill(sep, 0.0, 1)  # opening separator: one fill launch of one float
                for _ in range(3):
                    fn()
                capi.tensor_fill(sep, 0.0, 1)  # closing separator
                torch.cuda.synchronize()
                order.append(f"{L.name}.{pname}")
        print(json.dumps({"traffic_order": order, "calls_per_group": 3, "algorithmic_bytes": {f"{L.name}.{p}": L.bytes[p] for L in layers for p in ("fwd", "dgrad", "wgrad")},
                          "separator": "a fill of 1 float before and after each group of three calls"}))
        return
    step_flops = sum(3 * L.mult * L.flops for L in layers)
    slice_entries = [e for L in layers for e in L.slice_entries()]
    slice_table = capi.slice_sum_table(slice_entries) if slice_entries else None

    def step():
        for L in layers:
            for _ in range(L.mult):
                L.fwd()
        for L in reversed(layers):
            for k in range(L.mult):
                if L.n_slices:
                    L.bwd_sliced(k)  # data gradient + weight-gradient slices of the layer in one launch
                else:
                    L.bwd()
        if slice_table is not None:
            capi.sum_slices_multi(slice_table)  # every layer's dW += its slices, one launch

    def step_three_call():
        """The reference's call sequence: conv per layer on the way forward, convDerive then convError per layer on the way back."""
        for L in layers:
            for _ in range(L.mult):
                L.fwd()
        for L in reversed(layers):
            for _ in range(L.mult):
                L.dgrad()
                L.wgrad()

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    dt = timed(step)
    dt3 = timed(step_three_call)
    three_call = {
        "value": step_flops * args.steps / dt3 / 1e12, "unit": "TFLOP/s", "ms_per_step": dt3 / args.steps * 1e3,
        "frac_fp32_mfma_peak": step_flops * args.steps / dt3 / 1e12 / PEAK_FP32_MFMA_TFLOPS,
        "images_per_s": BATCH * args.steps / dt3, "steps": args.steps,
        "calls": "crb_conv_fwd, crb_conv_dgrad, crb_conv_wgrad per layer (the reference's conv / convDerive / convError sequence)",
    }

    # cold variants: every layer instance on buffers of its own
    for L in layers:
        L.make_cold_sets(torch, dev)

    def step_cold():
        for L in layers:
            for k in range(L.mult):
                L.fwd_cold(k)
        for L in reversed(layers):
            for k in range(L.mult):
                if L.n_slices:
                    L.bwd_sliced_cold(k)
                else:
                    L.bwd_cold(k)
        if slice_table is not None:
            capi.sum_slices_multi(slice_table)

    def step_three_call_cold():
        for L in layers:
            for k in range(L.mult):
                L.fwd_cold(k)
        for L in reversed(layers):
            for k in range(L.mult):
                L.dgrad_wgrad_cold(k)

    dt_cold, dt3_cold = timed(step_cold), timed(step_three_call_cold)
    cold_bytes = sum(sum(t.numel() * 4 for t in st) for L in layers for st in L.sets)
    for L in layers:
        L.sets = None
    torch.cuda.empty_cache()
    ms_per_step = dt / args.steps * 1e3
    tflops = step_flops * args.steps / dt / 1e12
    images_per_s = BATCH * args.steps / dt

    # instrumented pass: per-(layer, pass) launch duration with events on the launch stream
    per = {}
    for L in layers:
        for pname, fn, fl, in_step in L.passes():
            ms = event_time_ms(torch, fn, reps=50)
            per[f"{L.name}.{pname}"] = {
                "ms": ms, "tflops": fl / ms / 1e9, "gbs": L.bytes[pname] / ms / 1e6, "mult": L.mult if in_step else 0,
                "flops": fl, "bytes": L.bytes[pname],
            }
    sum_ms = event_time_ms(torch, lambda: capi.sum_slices_multi(slice_table), reps=20) if slice_table is not None else 0.0
    dom = max(per, key=lambda k: per[k]["ms"] * per[k]["mult"])
    d = per[dom]
    hbm_bytes, hbm_commit, hbm_src_hash = measured_hbm_bytes()
    from crusaderbackend_amd import bench_report

    if hbm_src_hash is None:
        src_note = "the profile records no kernel source hash"
    elif hbm_src_hash == bench_report.csrc_hash():
        src_note = "kernel sources (crusaderbackend_amd/csrc) unchanged since"
    else:
        src_note = "WARNING: kernel sources (crusaderbackend_amd/csrc) have changed since the counters were taken (hash %s then, %s now)" % (
            hbm_src_hash, bench_report.csrc_hash())
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": d["tflops"], "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
        "frac": d["tflops"] / PEAK_FP32_MFMA_TFLOPS, "traffic": hbm_bytes.get(dom),
        "traffic_unit": "bytes per call (FETCH_SIZE and WRITE_SIZE of rocprofv3 --pmc, scaled against a copy kernel)",
        "traffic_source": "profiles/resnet56_conv_step_b128.md, table 'HBM bytes per call', counters taken at commit %s (not measured by this run); %s" % (hbm_commit, src_note),
        "algorithmic_bytes": d["bytes"],
        "flops_per_launch": d["flops"], "avg_launch_ms": d["ms"],
        "share_of_step": d["ms"] * d["mult"] / sum(v["ms"] * v["mult"] for v in per.values()),
    }
    kern_sum_ms = sum(v["ms"] * v["mult"] for v in per.values()) + sum_ms

    # headline GEMM target: 4096^3 sgemm
    n = 4096
    A = torch.rand(n, n, device=dev) * 2 - 1
    B = torch.rand(n, n, device=dev) * 2 - 1
    C = torch.empty(n, n, device=dev)
    # three averages of ten launches: the first follows the allocations above, with the device clock still ramping up, and
    # reads several per cent high; the smallest is reported and all three are kept in `extra`
    gemm_runs = [event_time_ms(torch, lambda: capi.sgemm_nn(A, B, C, n, n, n), reps=10) for _ in range(3)]
    gemm_ms, gemm_ms_mean = min(gemm_runs), sum(gemm_runs) / len(gemm_runs)
    gemm_tflops = 2.0 * n ** 3 / gemm_ms / 1e9
    del A, B, C
    torch.cuda.empty_cache()

    # the other benchmark configurations, one figure each (the full per-call tables: --report)
    configs = None if args.no_configs else bench_report.compact(torch, capi, dev, event_time_ms, Layer)

    clock_khz = device_clock_khz()

    out = {
        "metric": "fp32 conv TFLOP/s, ResNet-56 conv layers fwd+dgrad+wgrad (also % FP32 MFMA peak, images/s in extra)",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ResNet-56 CIFAR conv shapes, fp32 NCHW, batch 128, 3x3 pad 1: 19x16->16@32, 17x32->32@16, "
                               "18x64->64@8, 16->32 s2, 32->64 s2; forward + dgrad + wgrad per layer (the two gradients of a layer "
                               "issued as one crb_conv_bwd_sliced call, the 55 layers' weight-gradient slices summed by one "
                               "crb_sum_slices_multi call at the end of the step)",
                   "batch": BATCH, "flops_per_step": step_flops},
        "roofline": roofline,
        "three_call_step": three_call,
        "extra": {
            "cold_ms_per_step": dt_cold / args.steps * 1e3, "cold_tflops": step_flops * args.steps / dt_cold / 1e12,
            "cold_three_call_ms_per_step": dt3_cold / args.steps * 1e3,
            "cold_three_call_tflops": step_flops * args.steps / dt3_cold / 1e12,
            "cold_distinct_operand_bytes": cold_bytes,
            "frac_fp32_mfma_peak": tflops / PEAK_FP32_MFMA_TFLOPS,
            "resnet56_conv_images_per_s": images_per_s,
            "resnet56_conv_images_per_s_kernel_only": BATCH / (kern_sum_ms / 1e3),
            "kernel_only_tflops": step_flops / kern_sum_ms / 1e9,
            "sgemm_4096_tflops": gemm_tflops, "sgemm_4096_ms": gemm_ms, "sgemm_4096_ms_runs": gemm_runs,
            "sgemm_4096_frac_peak": gemm_tflops / PEAK_FP32_MFMA_TFLOPS,
            "sgemm_4096_ms_mean": gemm_ms_mean, "sgemm_4096_tflops_mean": 2.0 * 4096 ** 3 / gemm_ms_mean / 1e9,
            "sgemm_4096_frac_peak_mean": 2.0 * 4096 ** 3 / gemm_ms_mean / 1e9 / PEAK_FP32_MFMA_TFLOPS,
            "slice_sum_all_layers_ms": sum_ms, "slice_sum_items": len(slice_entries),
            "per_kernel": {k: {"ms": round(v["ms"], 5), "tflops": round(v["tflops"], 2), "gbs": round(v["gbs"], 1)}
                           for k, v in per.items()},
            "full_network_steps_cpp_host": full_net,
            "device": props.name, "cus": props.multi_processor_count, "clock_mhz": clock_khz / 1e3,
            # 256 flop per clock per CU on the fp32 matrix pipe, at the peak clock the device reports
            "peak_from_reported_clock_tflops": props.multi_processor_count * clock_khz * 1e3 * 256 / 1e12,
        },
    }
    if configs is not None:
        out["configs"] = configs
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(RESNET56)
    if args.report:
        rep = bench_report.run(torch, capi, dev, event_time_ms, Layer)
        with open(args.report, "w") as f:
            json.dump(rep, f, indent=1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
