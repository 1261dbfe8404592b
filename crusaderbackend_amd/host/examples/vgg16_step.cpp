// VGG-16 (CIFAR variant) built with the seann host layer exactly as a user of the reference would write it:
// a Sequential of Conv2D / ReLU / MaxPool2D / Linear / Softmax with a momentum optimizer and the cross-entropy loss.
// Runs training steps (forward, backward, learn) on synthetic data and prints one JSON line with the step time in the
// reference's blocking mode (host synchronisation after every operator) and in the non-blocking mode (one
// synchronisation per step).
//   usage: vgg16_step [batch=128] [steps=10] [trace]     (trace: print the loss of every step of a short run first)
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../seann/containers/Sequential.h"
#include "../seann/operands/Conv2D.h"
#include "../seann/operands/Elementwise.h"
#include "../seann/operands/Linear.h"

using namespace seann;

static bool g_fused = false;  // use Sequential::learnFused

static void learn(Sequential &net) {
    if (g_fused)
        net.learnFused();
    else
        net.learn();
}

static double time_steps(Sequential &net, Tensor *X, Tensor *L, int steps) {
    for (int i = 0; i < 2; ++i) {  // warm-up
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
    const uint32 batch = argc > 1 ? uint32(std::atoi(argv[1])) : 128;
    const int steps = argc > 2 ? std::atoi(argv[2]) : 10;
    std::vector<OperandBase *> ops;
    uint32 C = 3, H = 32;
    double flops = 0;
    const int cfg[] = {64, 64, 0, 128, 128, 0, 256, 256, 256, 0, 512, 512, 512, 0, 512, 512, 512, 0};
    for (int oc : cfg) {
        if (oc == 0) {
            ops.push_back(new MaxPool2D(2, 2, 2, 2));
            H /= 2;
        } else {
            ops.push_back(new Conv2D(shape4(uint32(oc), C, 3, 3), 1, 1, 1, 1, true));
            ops.push_back(new ReLU());
            flops += 3 * 2.0 * batch * oc * H * H * C * 9;
            C = uint32(oc);
        }
    }
    ops.push_back(new Linear(512));
    ops.push_back(new ReLU());
    ops.push_back(new Linear(10));
    ops.push_back(new Softmax());
    flops += 3 * 2.0 * batch * (512.0 * 512 + 512 * 10);

    OPTIMIZER_MOMENTUM opt(2e-4f, 0.9f);  // gradients are sums over the batch (the loss gradient carries no 1/N), so the rate is small
    Sequential net(shape4(batch, 3, 32, 32), ops);
    net.construct(&opt);
    net.setLoss(crossEntropyLoss, crossEntropyCalc);
    net.randInit();

    Tensor *X = Tensor::create(batch, 3, 32, 32)->randNormal(0.f, 1.f, 40);
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
    std::printf("{\"workload\": \"VGG-16 CIFAR training step through seann::Sequential (C++ host layer)\", \"batch\": %u, "
                "\"steps\": %d, \"ms_per_step_blocking\": %.3f, \"ms_per_step_nonblocking\": %.3f, \"conv_fc_gflop\": %.2f, "
                "\"tflops_nonblocking\": %.2f, \"images_per_s_nonblocking\": %.1f, \"ms_per_step_pruned_fused\": %.3f, "
                "\"tflops_pruned_fused\": %.2f, \"images_per_s_pruned_fused\": %.1f, \"loss_after\": %.4f}\n",
                batch, steps, ms_blocking, ms_async, flops / 1e9, flops / ms_async / 1e9, batch / ms_async * 1e3, ms_fast,
                flops / ms_fast / 1e9, batch / ms_fast * 1e3, double(loss));
    return 0;
}
