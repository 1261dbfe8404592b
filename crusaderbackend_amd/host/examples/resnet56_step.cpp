// ResNet-56 (CIFAR) with the topology of the reference's archived model, built with the seann host layer: stem
// 3->16 + BatchNorm + ReLU; 9 identity blocks at 16 channels; a transition block (16->16, 16->32 stride 2, 1x1 stride-2
// projection shortcut); 8 identity blocks at 32; a transition block to 64; 9 identity blocks at 64; Linear 4096->1024->10;
// Softmax; momentum optimizer; cross-entropy. Every block is conv-BN-ReLU-conv-BN between a pair of ShortcutEndpoints,
// followed by ReLU. Convolutions carry no bias.
// Runs training steps (forward, backward, learn) on synthetic data and prints one JSON line: step time in the blocking
// mode of the reference (host synchronisation after every operator) and with one synchronisation per step.
//   usage: resnet56_step [batch=64] [steps=10] [trace]
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../seann/containers/Sequential.h"
#include "../seann/operands/Conv2D.h"
#include "../seann/operands/Elementwise.h"
#include "../seann/operands/Linear.h"
#include "../seann/operands/ShortcutEndpoint.h"

using namespace seann;

static double g_conv_flops = 0;  // forward flops of all convolutions / dense layers for one sample

static Conv2D *conv3x3(uint32 oc, uint32 ic, uint32 stride, uint32 outHW) {
    g_conv_flops += 2.0 * oc * outHW * outHW * ic * 9;
    return new Conv2D(shape4(oc, ic, 3, 3), stride, stride, 1, 1, false);
}

static void block(std::vector<OperandBase *> &ops, uint32 &uuid, uint32 ic, uint32 oc, uint32 inHW) {
    const uint32 stride = ic == oc ? 1 : 2, outHW = inHW / stride;
    ops.push_back(new ShortcutEndpoint(false, uuid, {}));
    ops.push_back(conv3x3(ic, ic, 1, inHW));
    ops.push_back(new BatchNorm());
    ops.push_back(new ReLU());
    ops.push_back(conv3x3(oc, ic, stride, outHW));
    ops.push_back(new BatchNorm());
    if (ic == oc) {
        ops.push_back(new ShortcutEndpoint(true, uuid, {}));
    } else {
        g_conv_flops += 2.0 * oc * outHW * outHW * ic;
        ops.push_back(new ShortcutEndpoint(true, uuid, {new Conv2D(shape4(oc, ic, 1, 1), 2, 2, 0, 0, false)}));
    }
    ops.push_back(new ReLU());
    ++uuid;
}

static bool g_fused = false;  // use Sequential::learnFused

static void learn(Sequential &net) {
    if (g_fused)
        net.learnFused();
    else
        net.learn();
}

static double time_steps(Sequential &net, Tensor *X, Tensor *L, int steps) {
    for (int i = 0; i < 2; ++i) {
        net.forward(X);
        net.backward(L);
        learn(net);
    }
    (void)hipDeviceSynchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) {
        net.forward(X);
        net.backward(L);
        learn(net);
    }
    (void)hipDeviceSynchronize();
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
}

int main(int argc, char **argv) {
    const uint32 batch = argc > 1 ? uint32(std::atoi(argv[1])) : 64;
    const int steps = argc > 2 ? std::atoi(argv[2]) : 10;
    std::vector<OperandBase *> ops;
    uint32 uuid = 1;
    ops.push_back(conv3x3(16, 3, 1, 32));
    ops.push_back(new BatchNorm());
    ops.push_back(new ReLU());
    for (int i = 0; i < 9; ++i) block(ops, uuid, 16, 16, 32);
    block(ops, uuid, 16, 32, 32);
    for (int i = 0; i < 8; ++i) block(ops, uuid, 32, 32, 16);
    block(ops, uuid, 32, 64, 16);
    for (int i = 0; i < 9; ++i) block(ops, uuid, 64, 64, 8);
    ops.push_back(new Linear(1024));
    ops.push_back(new Linear(10));
    ops.push_back(new Softmax());
    g_conv_flops += 2.0 * (4096.0 * 1024 + 1024 * 10);

    // gradients are sums over the batch (the loss gradient carries no 1/N): the archived model uses 0.01 / 64
    OPTIMIZER_MOMENTUM opt(0.01f / 64.0f, 0.9f);
    Sequential net(shape4(batch, 3, 32, 32), ops);
    net.construct(&opt);
    net.setLoss(crossEntropyLoss, crossEntropyCalc);
    net.randInit();

    Tensor *X = Tensor::create(batch, 3, 32, 32)->randNormal(0.f, 1.f, 56);
    Tensor *hl = Tensor::createHost(shape4(batch, 1, 10, 1));
    for (uint32 i = 0; i < batch * 10; ++i) hl->elements[i] = 0.f;
    for (uint32 n = 0; n < batch; ++n) hl->elements[n * 10 + (n * 7 + 3) % 10] = 1.f;
    Tensor *L = hl->toDevice();
    Tensor *lossBuf = Tensor::create(net.netY->A->dims);

    if (argc > 3) {
        for (int i = 0; i < 8; ++i) {
            net.forward(X);
            std::printf("step %d loss/sample %.5f\n", i, double(net.lossFW(net.netY, L, lossBuf)) / batch);
            net.backward(L);
            net.learn();
        }
    }
    setBlocking(true);
    const double ms_blocking = time_steps(net, X, L, steps);
    setBlocking(false);
    const double ms_async = time_steps(net, X, L, steps);
    // the same network with the optional shortcuts: streamlined graph, one launch for all momentum updates
    net.streamline();
    g_fused = true;
    const double ms_fast = time_steps(net, X, L, steps);
    g_fused = false;
    setBlocking(true);
    net.forward(X);
    const float loss = net.lossFW(net.netY, L, lossBuf);
    const double flops = 3.0 * g_conv_flops * batch;  // forward + data gradient + weight gradient
    std::printf("{\"workload\": \"ResNet-56 CIFAR training step (archived topology) through seann::Sequential\", \"batch\": %u, "
                "\"operands\": %zu, \"steps\": %d, \"ms_per_step_blocking\": %.3f, \"ms_per_step_nonblocking\": %.3f, "
                "\"conv_fc_gflop_per_step\": %.2f, \"tflops_nonblocking\": %.2f, \"images_per_s_nonblocking\": %.1f, "
                "\"images_per_s_blocking\": %.1f, \"ms_per_step_pruned_fused\": %.3f, \"images_per_s_pruned_fused\": %.1f, "
                "\"tflops_pruned_fused\": %.2f, \"loss_per_sample_after\": %.4f}\n",
                batch, ops.size(), steps, ms_blocking, ms_async, flops / 1e9, flops / ms_async / 1e9, batch / ms_async * 1e3,
                batch / ms_blocking * 1e3, ms_fast, batch / ms_fast * 1e3, flops / ms_fast / 1e9, double(loss) / batch);
    return 0;
}
