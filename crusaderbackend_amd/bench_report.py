"""Extended timing report over every benchmark configuration (used by ``bench.py --report FILE``).

Each entry: launch duration from HIP events on the launch stream (average of back-to-back launches), nominal
flops, algorithmic bytes (each operand read once, output written once), TFLOP/s, GB/s and the fraction of the
roofline that bounds the shape (FP32 matrix peak above ~19.7 flop/B, HBM bandwidth below).
"""
import hashlib
import math
import os

PEAK_TF = 157.3
PEAK_GBS = 8000.0
RIDGE = PEAK_TF * 1e3 / PEAK_GBS  # flop per byte
COLD_FOOTPRINT = 640e6  # bytes of distinct operands cycled through for the cold-cache figures


def csrc_hash():
    """sha256 over the kernel sources (crusaderbackend_amd/csrc: *.h, *.hip, *.cpp, Makefile, in name order), first 16 hex
    digits. Profile summaries that hold hardware-counter figures record it, so that a reader of those figures (bench.py's
    roofline.traffic) can tell whether the kernels have changed since the counters were taken."""
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(d)):
        if name.endswith((".h", ".hip", ".cpp")) or name == "Makefile":
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def _entry(name, ms, flops, nbytes):
    """`ms`: a time, or (smallest, mean) of the three averages of a row."""
    ms, ms_mean = ms if isinstance(ms, tuple) else (ms, ms)
    ai = flops / nbytes
    tf, gbs = flops / ms / 1e9, nbytes / ms / 1e6
    bound = "mfma" if ai >= RIDGE else "hbm"
    frac = tf / PEAK_TF if bound == "mfma" else gbs / PEAK_GBS
    return {"name": name, "us": round(ms * 1e3, 2), "us_mean": round(ms_mean * 1e3, 2), "gflop": round(flops / 1e9, 3),
            "mbytes": round(nbytes / 1e6, 2), "ai": round(ai, 1), "tflops": round(tf, 2), "gbs": round(gbs, 1), "bound": bound,
            "frac": round(frac, 4)}


VGG16_CONVS = [(3, 32, 64), (64, 32, 64), (64, 16, 128), (128, 16, 128), (128, 8, 256), (256, 8, 256), (256, 8, 256),
               (256, 4, 512), (512, 4, 512), (512, 4, 512), (512, 2, 512), (512, 2, 512), (512, 2, 512)]  # (IC, H, OC), 3x3 pad 1


def _settled(torch, capi, event_time_ms, fn, reps):
    """One row's time: the call is frozen (argument conversion done once: a plain wrapper call costs the host 3.5-4.5 us,
    more than the shortest kernels take), repeated until the timed region is at least a millisecond, three such averages.
    Returns (smallest, mean). Rows follow tensor allocation and host work during which the device clock drops, and its
    ramp back up takes tens of milliseconds (a dense layer timed right after its tensors were made read 13 % longer than
    the same call timed a little later), so a row first runs untimed for about 20 ms."""
    f = capi.frozen(fn)
    ms = event_time_ms(torch, f, reps=reps)
    event_time_ms(torch, f, reps=max(1, min(8000, int(20.0 / max(ms, 1e-4)))), warm=0)
    if ms * reps < 1.0:
        reps = min(4000, int(1.0 / ms) + 1)
    runs = [event_time_ms(torch, f, reps=reps) for _ in range(3)]
    return min(runs), sum(runs) / len(runs)


def _densenet_pairs(torch, capi, dev, Layer, device_rng=False):
    """The 48 bottleneck pairs of DenseNet-BC-100 (k = 12) at batch 64 (seann/operands/prefabs/DenseBlock.cuh:42-61: 1x1 IC -> 48
    then 3x3 48 -> 12, IC = 24 + 12 i @32x32, 108 + 12 i @16x16, 150 + 12 i @8x8, i = 0..15; archive/Densenet100:2-34), every
    layer on tensors of its own."""
    pairs = []
    for (H, base) in ((32, 24), (16, 108), (8, 150)):
        for i in range(16):
            IC = base + 12 * i
            pairs.append((Layer(torch, capi, dev, f"1x1_{IC}-48@{H}", IC, H, 48, 1, 1, seed=300 + i, batch=64, F=1, pad=0, bias=True, device_rng=device_rng),
                          Layer(torch, capi, dev, f"3x3_48-12@{H}", 48, H, 12, 1, 1, seed=400 + i, batch=64, F=3, pad=1, bias=True, device_rng=device_rng)))
    return pairs


def _densenet_step(torch, capi, event_time_ms, pairs):
    """Config 4 as a whole: forward in network order, then conv / convDerive / convError as separate calls per layer in
    reverse order; also the 1x1 layers alone and the 3x3 layers alone."""
    def dn_step(kinds):
        def run():
            for pw, c3 in pairs:
                if "1x1" in kinds:
                    pw.fwd()
                if "3x3" in kinds:
                    c3.fwd()
            for pw, c3 in reversed(pairs):
                if "3x3" in kinds:
                    c3.dgrad(), c3.wgrad()
                if "1x1" in kinds:
                    pw.dgrad(), pw.wgrad()
        return run

    def work(idx):
        return (sum(3 * p[idx].flops for p in pairs), sum(p[idx].bytes["fwd"] + p[idx].bytes["dgrad"] + p[idx].bytes["wgrad"] for p in pairs))

    # The same work as a training step needs it: per layer the forward call and ONE backward call that leaves the weight
    # gradient as slices (crb_conv_bwd_sliced), and one crb_sum_slices_multi over all 96 layers at the end of the step.
    sliced = [L for p in pairs for L in p if L.n_slices]
    table = capi.slice_sum_table([e for L in sliced for e in L.slice_entries()]) if sliced else None

    def streamlined():
        for pw, c3 in pairs:
            pw.fwd(), c3.fwd()
        for pw, c3 in reversed(pairs):
            for L in (c3, pw):
                if L.n_slices:
                    L.bwd_sliced(0)
                else:
                    L.bwd()
        if table is not None:
            capi.sum_slices_multi(table)

    sl_ms = min(event_time_ms(torch, streamlined, reps=5, warm=2) for _ in range(2))

    all_ms = min(event_time_ms(torch, dn_step(("1x1", "3x3")), reps=5, warm=2) for _ in range(2))
    pw_ms = min(event_time_ms(torch, dn_step(("1x1",)), reps=5, warm=2) for _ in range(2))
    c3_ms = min(event_time_ms(torch, dn_step(("3x3",)), reps=5, warm=2) for _ in range(2))
    (pw_fl, pw_by), (c3_fl, c3_by) = work(0), work(1)
    return {
        "workload": "DenseNet-BC-100 (k = 12) convolution layers, batch 64: 48 x (1x1 IC->48, 3x3 48->12), fwd + dgrad + wgrad as separate calls",
        "us": round(all_ms * 1e3, 1), "gflop": round((pw_fl + c3_fl) / 1e9, 2), "mbytes": round((pw_by + c3_by) / 1e6, 1),
        "tflops": round((pw_fl + c3_fl) / all_ms / 1e9, 2), "images_per_s": round(64 / all_ms * 1e3, 1),
        "pointwise_us": round(pw_ms * 1e3, 1), "pointwise_mbytes": round(pw_by / 1e6, 1), "pointwise_gbs": round(pw_by / pw_ms / 1e6, 1),
        "pointwise_frac_hbm": round(pw_by / pw_ms / 1e6 / PEAK_GBS, 4), "pointwise_tflops": round(pw_fl / pw_ms / 1e9, 2),
        "conv3x3_us": round(c3_ms * 1e3, 1), "conv3x3_gflop": round(c3_fl / 1e9, 2), "conv3x3_tflops": round(c3_fl / c3_ms / 1e9, 2),
        "conv3x3_frac_mfma": round(c3_fl / c3_ms / 1e9 / PEAK_TF, 4),
        "one_backward_call_us": round(sl_ms * 1e3, 1), "one_backward_call_tflops": round((pw_fl + c3_fl) / sl_ms / 1e9, 2),
        "one_backward_call_images_per_s": round(64 / sl_ms * 1e3, 1), "one_backward_call_layers_sliced": len(sliced),
    }


def _dense_rows(torch, capi, dev, settled):
    """Config 5: dense sweep (batch 256, 4096 <-> 4096) through linear* and the raw GEMM forms, plus tall-skinny."""
    def rnd(*shape):
        return torch.rand(*shape, device=dev) * 2 - 1

    rows = []
    b, n = 256, 4096
    X, W, bias = rnd(b, n), rnd(n, n), rnd(n)
    Y, dX, dW, dB = torch.empty(b, n, device=dev), torch.empty(b, n, device=dev), torch.zeros(n, n, device=dev), torch.zeros(n, device=dev)
    fl, by = 2.0 * b * n * n, 4.0 * (2 * b * n + n * n)
    for nm, fn in (("linear (Y=X*W^T+b)", lambda: capi.linear_fwd(X, W, bias, Y, b, n, n)),
                   ("linearXGrad (dX=dY*W)", lambda: capi.linear_dgrad(X, W, dX, b, n, n)),
                   ("linearParamGrad (dW+=dY^T*X)", lambda: capi.linear_wgrad(X, X, dW, dB, b, n, n)),
                   ("sgemmNT 256x4096x4096", lambda: capi.sgemm_nt(X, W, Y, b, n, n)),
                   ("sgemm 256x4096x4096", lambda: capi.sgemm_nn(X, W, Y, b, n, n)),
                   ("sgemmTN 4096x4096x256", lambda: capi.sgemm_tn(X, X, dW, n, n, b))):
        rows.append(_entry(nm, settled(fn, 20), fl, by))
    M, K, N = 32768, 576, 64
    A, B, C = rnd(M, K), rnd(K, N), torch.empty(M, N, device=dev)
    rows.append(_entry("sgemm tall-skinny 32768x64x576", settled(lambda: capi.sgemm_nn(A, B, C, M, N, K), 20),
                       2.0 * M * N * K, 4.0 * (M * K + K * N + M * N)))
    return rows


def _vgg_fc_rows(torch, capi, dev, settled):
    def rnd(*shape):
        return torch.rand(*shape, device=dev) * 2 - 1

    rows = []
    for (IN, OUT) in ((512, 512), (512, 10)):
        b = 128
        X, W, bias = rnd(b, IN), rnd(OUT, IN), rnd(OUT)
        Y, dY, dX, dW, dB = (torch.empty(b, OUT, device=dev), rnd(b, OUT), torch.empty(b, IN, device=dev),
                             torch.zeros(OUT, IN, device=dev), torch.zeros(OUT, device=dev))
        fl, by = 2.0 * b * IN * OUT, 4.0 * (b * IN + IN * OUT + b * OUT)
        # prepared calls: these kernels are shorter than the argument conversion of a plain ctypes call
        f_fwd = capi.prepared("crb_linear_fwd", X, W, bias, Y, b, IN, OUT, 0, None)
        f_dgrad = capi.prepared("crb_linear_dgrad", dY, W, dX, b, IN, OUT, None)
        f_wgrad = capi.prepared("crb_linear_wgrad", dY, X, dW, dB, b, IN, OUT, None)
        rows.append(_entry(f"fc{IN}-{OUT}.fwd", settled(f_fwd, 100), fl, by))
        rows.append(_entry(f"fc{IN}-{OUT}.dgrad", settled(f_dgrad, 100), fl, by))
        rows.append(_entry(f"fc{IN}-{OUT}.wgrad", settled(f_wgrad, 100), fl, by))
    return rows


def _row_sum(rows):
    us, gf = sum(e["us"] for e in rows), sum(e["gflop"] for e in rows)
    return {"ms": round(us / 1e3, 4), "tflops": round(gf / max(us, 1e-9) * 1e3, 2), "bound": "mfma",
            "frac": round(gf / max(us, 1e-9) * 1e3 / PEAK_TF, 4), "calls": len(rows)}


def compact(torch, capi, dev, event_time_ms, Layer):
    """One figure (or a few) per benchmark configuration other than the headline one, for the default bench line: a few
    seconds of GPU time. Same timing method and byte / flop accounting as the full report."""
    def settled(fn, reps):
        return _settled(torch, capi, event_time_ms, fn, reps)

    def pick(e):
        return {k: e[k] for k in ("us", "us_mean", "tflops", "gbs", "bound", "frac")}

    out = {}
    n = 1024
    A, B, C = (torch.rand(n, n, device=dev) * 2 - 1 for _ in range(3))
    out["1_sgemm_1024^3"] = pick(_entry("", settled(lambda: capi.sgemm_nn(A, B, C, n, n, n), 20), 2.0 * n ** 3, 12.0 * n * n))
    del A, B, C
    # config 3: every convolution and dense-layer call of one VGG-16 training step (fwd + dgrad + wgrad, bias fused), summed
    rows = []
    for i, (ic, h, oc) in enumerate(VGG16_CONVS):
        L = Layer(torch, capi, dev, f"c{i + 1}", ic, h, oc, 1, 1, seed=100 + i, batch=128, F=3, pad=1, bias=True, device_rng=True)
        for pname, fn, fl, _ in L.passes():
            if pname in ("fwd", "dgrad", "wgrad"):
                rows.append(_entry(pname, settled(fn, 30 if L.flops < 2e9 else 10), fl, L.bytes[pname]))
        del L
    rows += _vgg_fc_rows(torch, capi, dev, settled)
    out["3_vgg16_conv_fc_step_b128"] = _row_sum(rows)
    out["3_vgg16_conv_fc_step_b128"]["what"] = "sum of the per-call times of 13 conv + 2 FC layers x (fwd, dgrad, wgrad)"
    torch.cuda.empty_cache()
    from .vgg16_step import Vgg16Step
    net = Vgg16Step(torch, capi, dev, batch=128)
    step_ms = min(event_time_ms(torch, net.step, reps=10, warm=3) for _ in range(2))
    out["3_vgg16_train_step_b128"] = {"ms": round(step_ms, 4), "tflops": round(net.flops / step_ms / 1e9, 2), "bound": "mfma",
                                      "frac": round(net.flops / step_ms / 1e9 / PEAK_TF, 4), "images_per_s": round(128 / step_ms * 1e3, 1),
                                      "what": "whole training step: every operator, loss and momentum update on real data flow"}
    del net
    torch.cuda.empty_cache()
    # config 4: the whole DenseNet-BC-100 convolution step
    pairs = _densenet_pairs(torch, capi, dev, Layer, device_rng=True)
    d = _densenet_step(torch, capi, event_time_ms, pairs)
    del pairs
    torch.cuda.empty_cache()
    out["4_densenet_bc100_conv_step_b64"] = {
        "ms": round(d["us"] / 1e3, 4), "tflops": d["tflops"], "images_per_s": d["images_per_s"],
        "pointwise": {"ms": round(d["pointwise_us"] / 1e3, 4), "gbs": d["pointwise_gbs"], "bound": "hbm", "frac": d["pointwise_frac_hbm"]},
        "conv3x3": {"ms": round(d["conv3x3_us"] / 1e3, 4), "tflops": d["conv3x3_tflops"], "bound": "mfma", "frac": d["conv3x3_frac_mfma"]},
        "one_backward_call_per_layer": {"ms": round(d["one_backward_call_us"] / 1e3, 4), "tflops": d["one_backward_call_tflops"],
                                        "images_per_s": d["one_backward_call_images_per_s"],
                                        "what": "crb_conv_fwd + crb_conv_bwd_sliced per layer, one crb_sum_slices_multi per step"},
        "what": "48 x (1x1 IC->48, 3x3 48->12), conv / convDerive / convError as separate calls, every layer on tensors of its own"}
    # config 5
    for e in _dense_rows(torch, capi, dev, settled):
        out["5_" + e["name"]] = pick(e)
    return out


def run(torch, capi, dev, event_time_ms, Layer):
    out = {"gemm": [], "resnet56": [], "vgg16": [], "densenet": [], "dense": [], "offgrid": []}

    def rnd(*shape):
        return torch.rand(*shape, device=dev) * 2 - 1

    def settled(fn, reps):
        return _settled(torch, capi, event_time_ms, fn, reps)

    # config 1 + target GEMM
    for n in (1024, 4096):
        A, B, C = rnd(n, n), rnd(n, n), torch.empty(n, n, device=dev)
        ms = settled(lambda: capi.sgemm_nn(A, B, C, n, n, n), 20 if n == 1024 else 10)
        out["gemm"].append(_entry(f"sgemm {n}^3", ms, 2.0 * n ** 3, 12.0 * n * n))

    def conv_entries(key, specs, batch, bias):
        for i, (name, IC, H, OC, F, s, p) in enumerate(specs):
            L = Layer(torch, capi, dev, name, IC, H, OC, s, 1, seed=100 + i, batch=batch, F=F, pad=p, bias=bias)
            entries = {}
            for pname, fn, fl, _ in L.passes():
                if pname in ("bwd", "bwd_sliced") and key != "resnet56":  # the one-call forms of both gradients: residual-network shapes
                    continue
                reps = 30 if L.flops < 2e9 else 10
                entries[pname] = _entry(f"{name}.{pname}", settled(fn, reps), fl, L.bytes[pname])
                out[key].append(entries[pname])
            # Bandwidth-bound shapes also get a cold-cache figure: the same call cycled over enough distinct buffer sets
            # (>= 640 MB in total, beyond L2 and the 256 MB memory-side cache) that no launch finds its operands cached.
            if any(e["bound"] == "hbm" for e in entries.values()):
                per_set = max(L.bytes.values())
                copies = min(int(COLD_FOOTPRINT // per_set) + 1, 64)
                ring = [L] + [Layer(torch, capi, dev, name, IC, H, OC, s, 1, seed=100 + i, batch=batch, F=F, pad=p, bias=bias)
                              for _ in range(copies - 1)]
                for pname in entries:
                    fns = [{p[0]: p[1] for p in R.passes()}[pname] for R in ring]
                    state = {"i": 0}

                    def cyc():
                        fns[state["i"] % len(fns)]()
                        state["i"] += 1

                    ms = event_time_ms(torch, cyc, reps=2 * len(fns), warm=len(fns))
                    e = entries[pname]
                    e["us_cold"] = round(ms * 1e3, 2)
                    e["gbs_cold"] = round(L.bytes[pname] / ms / 1e6, 1)
                    e["cold_sets"] = len(fns)
                del ring
            del L
            torch.cuda.empty_cache()

    # config 2: the five 3x3 shapes + stem + the two 1x1 stride-2 shortcuts
    conv_entries("resnet56", [("16-16@32", 16, 32, 16, 3, 1, 1), ("32-32@16", 32, 16, 32, 3, 1, 1),
                              ("64-64@8", 64, 8, 64, 3, 1, 1), ("16-32s2", 16, 32, 32, 3, 2, 1),
                              ("32-64s2", 32, 16, 64, 3, 2, 1), ("stem3-16@32", 3, 32, 16, 3, 1, 1),
                              ("sc16-32_1x1s2", 16, 32, 32, 1, 2, 0), ("sc32-64_1x1s2", 32, 16, 64, 1, 2, 0)], 128, False)

    # config 3: VGG-16 (CIFAR) conv layers, bias fused, batch 128
    conv_entries("vgg16", [(f"c{i + 1}_{ic}-{oc}@{h}", ic, h, oc, 3, 1, 1) for i, (ic, h, oc) in enumerate(VGG16_CONVS)], 128, True)
    out["vgg16"] += _vgg_fc_rows(torch, capi, dev, settled)

    # config 4: DenseNet-BC-100 (k = 12), batch 64: first / middle / last bottleneck of each stage + the 3x3
    dn = []
    for (H, base) in ((32, 24), (16, 108), (8, 150)):
        for i in (0, 8, 15):
            dn.append((f"1x1_{base + 12 * i}-48@{H}", base + 12 * i, H, 48, 1, 1, 0))
        dn.append((f"3x3_48-12@{H}", 48, H, 12, 3, 1, 1))
    conv_entries("densenet", dn, 64, True)

    # Layers off the benchmark networks' width grid (no configuration of the baseline; the geometries of ImageNet-style residual
    # networks, a 5x5 layer, a 3x3 layer without padding, a 4x4 stride-2 layer, a 7x7 stride-2 stem), batch 32
    conv_entries("offgrid", [("64-64@56", 64, 56, 64, 3, 1, 1), ("128-128@28", 128, 28, 128, 3, 1, 1), ("256-256@14", 256, 14, 256, 3, 1, 1),
                             ("512-512@7", 512, 7, 512, 3, 1, 1), ("64-128@56s2", 64, 56, 128, 3, 2, 1),
                             ("128-256@28s2", 128, 28, 256, 3, 2, 1), ("256-512@14s2", 256, 14, 512, 3, 2, 1),
                             ("sc64-128@56_1x1s2", 64, 56, 128, 1, 2, 0), ("5x5_64-64@28p2", 64, 28, 64, 5, 1, 2),
                             ("3x3_64-64@30p0", 64, 30, 64, 3, 1, 0), ("4x4s2_64-128@32p1", 64, 32, 128, 4, 2, 1),
                             ("7x7s2_3-64@224p3", 3, 224, 64, 7, 2, 3)], 32, False)

    # config 4 as a whole: the convolution work of one DenseNet-BC-100 training step at batch 64
    pairs = _densenet_pairs(torch, capi, dev, Layer)
    out["densenet_full_step"] = _densenet_step(torch, capi, event_time_ms, pairs)
    del pairs
    torch.cuda.empty_cache()

    # config 5: dense sweep (batch 256, 4096 <-> 4096) through linear* and the raw GEMM forms, plus tall-skinny
    out["dense"] = _dense_rows(torch, capi, dev, settled)

    # elementwise / reduction operators at the sizes the VGG-16 step runs them (all bandwidth-bound; flops counted as 0)
    out["elementwise"] = []

    def ew(name, fn, nbytes, reps=30):
        ms, ms_mean = settled(fn, reps)
        out["elementwise"].append({"name": name, "us": round(ms * 1e3, 2), "us_mean": round(ms_mean * 1e3, 2), "gflop": 0.0, "mbytes": round(nbytes / 1e6, 2), "ai": 0.0,
                                   "tflops": 0.0, "gbs": round(nbytes / ms / 1e6, 1), "bound": "hbm",
                                   "frac": round(nbytes / ms / 1e6 / PEAK_GBS, 4)})

    for (C, H) in ((64, 32), (256, 8)):
        n = 128 * C * H * H
        X, Y, dY = rnd(n), torch.empty(n, device=dev), rnd(n)
        ew(f"relu 128x{C}x{H}x{H}", lambda: capi.relu_fwd(X, Y, n), 8.0 * n)
        ew(f"reluGradFast 128x{C}x{H}x{H}", lambda: capi.relu_bwd(X, dY, Y, n), 12.0 * n)
        P, rec = torch.empty(n // 4, device=dev), torch.empty(n, device=dev)
        ew(f"maxPool 2x2 128x{C}x{H}x{H}", lambda: capi.maxpool_fwd(X, P, rec, 128 * C, H, H, 2, 2, 2, 2), 4.0 * (2 * n + n // 4))
        ew(f"maxPoolBack 2x2 128x{C}x{H}x{H}", lambda: capi.maxpool_bwd(Y, P, rec, 128 * C, H, H, 2, 2, 2, 2), 4.0 * (3 * n + n // 4))
        del X, Y, dY, P, rec
    n = 512 * 512 * 9
    Wt, G, M = rnd(n), rnd(n), rnd(n)
    ew("momentumApply + decay 512x512x3x3", lambda: capi.momentum_apply(Wt, G, M, n, 0.01, 0.9, 0.9995), 24.0 * n)
    A, S, L = rnd(128, 10), torch.empty(128, 10, device=dev), torch.zeros(128, 10, device=dev)
    loss = torch.empty(1, device=dev)
    ew("softmax 128x10", lambda: capi.softmax(A, S, 128, 10), 8.0 * 1280)
    ew("crossEntropyCalc 128x10", lambda: capi.cross_entropy_loss(S, L, None, loss, 1280), 8.0 * 1280)
    del Wt, G, M
    # dataset bytes -> network input, one batch of the archived CIFAR programs (6400 images): 1 byte read, 4 written per value
    nimg = 6400
    raw = torch.randint(0, 256, (nimg, 3, 32, 32), dtype=torch.uint8, device=dev)
    Xf = torch.empty(nimg, 3, 32, 32, device=dev)
    aug = capi.image_aug_table(torch, dev, [((i % 9) - 4, ((i // 9) % 9) - 4, i % 4) for i in range(nimg)])
    nb = 5.0 * raw.numel()
    ew("bytes->float 6400x3x32x32", lambda: capi.images_from_bytes(raw, Xf, nimg, 3, 32, 32), nb)
    ew("bytes->float + UniformNorm 6400x3x32x32", lambda: capi.images_from_bytes(raw, Xf, nimg, 3, 32, 32, capi.NORM_UNIFORM, 0.0, 1.0), nb)
    ew("bytes->float + DistribNorm 6400x3x32x32", lambda: capi.images_from_bytes(raw, Xf, nimg, 3, 32, 32, capi.NORM_DISTRIBUTION, 0.0, 1.0), nb)
    ew("bytes->float + UniformNorm + mirror/shift 6400x3x32x32",
       lambda: capi.images_from_bytes(raw, Xf, nimg, 3, 32, 32, capi.NORM_UNIFORM, 0.0, 1.0, aug=aug), nb)
    del raw, Xf, aug

    # config 3 end to end: the whole training step (every operator, real data flow, momentum update), batch 128
    from .vgg16_step import Vgg16Step
    net = Vgg16Step(torch, capi, dev, batch=128)
    step_ms = event_time_ms(torch, net.step, reps=10, warm=3)
    fwd_ms = event_time_ms(torch, net.forward, reps=10, warm=2)
    bwd_ms = event_time_ms(torch, net.backward, reps=10, warm=2)
    upd_ms = event_time_ms(torch, net.update, reps=10, warm=2)
    out["vgg16_full_step"] = {"us": round(step_ms * 1e3, 1), "forward_us": round(fwd_ms * 1e3, 1), "backward_us": round(bwd_ms * 1e3, 1),
                              "update_us": round(upd_ms * 1e3, 1), "conv_fc_gflop": round(net.flops / 1e9, 2),
                              "tflops": round(net.flops / step_ms / 1e9, 2), "images_per_s": round(128 / step_ms * 1e3, 1),
                              "frac_fp32_mfma_peak": round(net.flops / step_ms / 1e9 / PEAK_TF, 4)}
    del net
    torch.cuda.empty_cache()

    # summary lines
    def total(key, suffix=None):
        es = [e for e in out[key] if suffix is None or e["name"].endswith(suffix)]
        return {"us": round(sum(e["us"] for e in es), 1), "gflop": round(sum(e["gflop"] for e in es), 2),
                "tflops": round(sum(e["gflop"] for e in es) / max(sum(e["us"] for e in es), 1e-9) * 1e3, 2)}

    out["summary"] = {"vgg16_conv_fc_train_step": total("vgg16"), "vgg16_fwd": total("vgg16", ".fwd"),
                      "vgg16_full_train_step": out["vgg16_full_step"], "densenet_bc100_conv_step": out["densenet_full_step"],
                      "peak_fp32_mfma_tflops": PEAK_TF, "peak_hbm_gbs": PEAK_GBS, "ridge_flop_per_byte": round(RIDGE, 2)}
    return out


def to_markdown(rep):
    lines = []
    for key in ("gemm", "resnet56", "vgg16", "densenet", "offgrid", "dense", "elementwise"):
        if key not in rep:
            continue
        lines += [f"### {key}", "", "| shape.pass | us (smallest of 3 averages) | us (mean of the 3) | GFLOP | MB | AI | TFLOP/s | GB/s | bound | fraction of roofline | cold-cache us | cold GB/s |",
                  "|---|---|---|---|---|---|---|---|---|---|---|---|"]
        for e in rep[key]:
            cold = f"{e['us_cold']} | {e['gbs_cold']}" if "us_cold" in e else " | "
            lines.append(f"| {e['name']} | {e['us']} | {e.get('us_mean', '')} | {e['gflop']} | {e['mbytes']} | {e['ai']} | {e['tflops']} | {e['gbs']} | {e['bound']} | {e['frac'] * 100:.1f} % | {cold} |")
        lines.append("")
    return "\n".join(lines)
