"""One full VGG-16 (CIFAR variant) training step driven through the C ABI: the measurement workload of the
"VGG-16 full train step" configuration and the end-to-end parity case.

Network: 3x3 pad-1 convolutions 64,64,M,128,128,M,256x3,M,512x3,M,512x3,M with bias, ReLU after each, 2x2 max pooling
at every M, then FC 512->512 + ReLU -> 10, softmax, cross-entropy; momentum update with L2 weight decay on the weights.
The order of calls is the reference's Sequential (seann/containers/Sequential.cu:43-47 forward, :79-85 backward with
xGrads then paramGrads per operand from last to first, :93-97 update): every operand's input gradient is computed,
the first convolution's included. ReLU is a separate pass, as in the reference (no fused epilogue is used here).

All device buffers are torch tensors; torch performs no arithmetic. `params()` copies the learnable state to numpy so
a CPU replica can be run on identical values.
"""
import math

CFG = (64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M")


class Vgg16Step:
    def __init__(self, torch, capi, dev, batch=128, image=32, classes=10, seed=40, lr=0.01, beta=0.9, l2=5e-4, cfg=CFG,
                 hidden=512):
        self.torch, self.capi, self.dev = torch, capi, dev
        self.batch, self.classes, self.lr, self.beta, self.l2 = batch, classes, lr, beta, l2
        gen = torch.Generator(device="cpu").manual_seed(seed)

        def dev_randn(*shape, std=1.0):
            return (torch.randn(*shape, generator=gen) * std).to(dev)

        def zeros(*shape):
            return torch.zeros(*shape, dtype=torch.float32, device=dev)

        self.x = dev_randn(batch, 3, image, image)
        labels = torch.randint(0, classes, (batch,), generator=gen)
        self.labels = torch.nn.functional.one_hot(labels, classes).to(torch.float32).to(dev)
        self.dx = zeros(batch, 3, image, image)

        # stages: ("conv", dict) / ("pool", dict); every dict holds its output value and the gradient w.r.t. it
        self.stages, self.learn = [], []
        C, H = 3, image
        for item in cfg:
            if item == "M":
                st = {"C": C, "IH": H, "out": zeros(batch, C, H // 2, H // 2), "dout": zeros(batch, C, H // 2, H // 2),
                      "rec": zeros(batch, C, H, H)}
                H //= 2
                self.stages.append(("pool", st))
            else:
                OC = item
                g = capi.ConvGeom.make(batch, C, H, H, OC, 3, 3, 1, 1, 1, 1)
                nbytes = capi.conv_wgrad_workspace_bytes(g)
                st = {"g": g, "IC": C, "OC": OC, "H": H,
                      "W": dev_randn(OC, C, 3, 3, std=math.sqrt(2.0 / (C * 9))), "b": dev_randn(OC, std=math.sqrt(2.0 / OC)),
                      "dW": zeros(OC, C, 3, 3), "dB": zeros(OC), "mW": zeros(OC, C, 3, 3), "mB": zeros(OC),
                      "z": zeros(batch, OC, H, H), "dz": zeros(batch, OC, H, H),
                      "out": zeros(batch, OC, H, H), "dout": zeros(batch, OC, H, H),
                      "ws": torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=dev) if nbytes else None}
                self.learn += [(st, "W", "dW", "mW", True), (st, "b", "dB", "mB", False)]
                self.stages.append(("conv", st))
                C = OC
        self.flat = C * H * H
        self.fc = []
        IN = self.flat
        for OUT, relu in ((hidden, True), (classes, False)):
            st = {"IN": IN, "OUT": OUT, "relu": relu,
                  "W": dev_randn(OUT, IN, std=math.sqrt(2.0 / IN)), "b": dev_randn(OUT, std=math.sqrt(2.0 / IN)),
                  "dW": zeros(OUT, IN), "dB": zeros(OUT), "mW": zeros(OUT, IN), "mB": zeros(OUT),
                  "z": zeros(batch, OUT), "dz": zeros(batch, OUT), "out": zeros(batch, OUT), "dout": zeros(batch, OUT)}
            self.learn += [(st, "W", "dW", "mW", True), (st, "b", "dB", "mB", False)]
            self.fc.append(st)
            IN = OUT
        self.probs = zeros(batch, classes)
        self.loss = zeros(1)
        n = capi.cross_entropy_scratch_floats(batch * classes)
        self.loss_scratch = zeros(max(n, 1))
        self.flops = self._flops()

    def _flops(self):
        f = 0.0
        for kind, st in self.stages:
            if kind == "conv":
                f += 3 * 2.0 * self.batch * st["OC"] * st["H"] * st["H"] * st["IC"] * 9
        for st in self.fc:
            f += 3 * 2.0 * self.batch * st["IN"] * st["OUT"]
        return f

    # ---- one step ---------------------------------------------------------------------------------------------------
    def forward(self):
        c, B = self.capi, self.batch
        cur = self.x
        for kind, st in self.stages:
            if kind == "conv":
                c.conv_fwd(st["W"], cur, st["z"], st["b"], st["g"])
                c.relu_fwd(st["z"], st["out"], st["z"].numel())
            else:
                c.maxpool_fwd(cur, st["out"], st["rec"], B * st["C"], st["IH"], st["IH"], 2, 2, 2, 2)
            cur = st["out"]
        for st in self.fc:
            c.linear_fwd(cur, st["W"], st["b"], st["z"], B, st["IN"], st["OUT"])
            if st["relu"]:
                c.relu_fwd(st["z"], st["out"], st["z"].numel())
                cur = st["out"]
            else:
                cur = st["z"]
        c.softmax(cur, self.probs, B, self.classes)
        c.cross_entropy_loss(self.probs, self.labels, self.loss_scratch, self.loss, B * self.classes)

    def backward(self):
        c, B = self.capi, self.batch
        last = self.fc[-1]
        c.cross_entropy_grad(self.probs, self.labels, last["dz"], B * self.classes)
        # dense layers, last to first; the gradient w.r.t. a layer's input lands in the producer's "dout"
        for i in range(len(self.fc) - 1, -1, -1):
            st = self.fc[i]
            src = self.fc[i - 1] if i > 0 else self.stages[-1][1]
            if st["relu"]:
                c.relu_bwd(st["z"], st["dout"], st["dz"], st["z"].numel())
            c.linear_dgrad(st["dz"], st["W"], src["dout"], B, st["IN"], st["OUT"])
            c.linear_wgrad(st["dz"], src["out"], st["dW"], st["dB"], B, st["IN"], st["OUT"])
        for i in range(len(self.stages) - 1, -1, -1):
            kind, st = self.stages[i]
            src_out = self.stages[i - 1][1]["out"] if i > 0 else self.x
            src_dout = self.stages[i - 1][1]["dout"] if i > 0 else self.dx
            if kind == "pool":
                c.maxpool_bwd(src_dout, st["dout"], st["rec"], B * st["C"], st["IH"], st["IH"], 2, 2, 2, 2)
            else:
                c.relu_bwd(st["z"], st["dout"], st["dz"], st["z"].numel())
                c.conv_dgrad(st["W"], st["dz"], src_dout, st["g"])
                c.conv_wgrad(st["dz"], src_out, st["dW"], st["g"], workspace=st["ws"])
                c.conv_bias_grad(st["dz"], st["dB"], B, st["OC"], st["H"] * st["H"])

    def update(self):
        for st, p, g, m, is_weight in self.learn:
            self.capi.momentum_apply(st[p], st[g], st[m], st[p].numel(), self.lr, self.beta,
                                     1.0 - self.l2 if is_weight else 1.0)

    def step(self):
        self.forward()
        self.backward()
        self.update()

    # ---- state exchange with a CPU replica ------------------------------------------------------------------------------
    def layers(self):
        return [st for kind, st in self.stages if kind == "conv"] + self.fc

    def params(self):
        return [{k: st[k].detach().cpu().numpy().copy() for k in ("W", "b", "dW", "dB", "mW", "mB")} for st in self.layers()]
