// Host-side tests of the C++ seblas / seann layer. Mode "host" needs no GPU (shape rules, exact division helper,
// shape-error translation, which all happen before any device work). Mode "gpu" drives the reference-shaped API
// end to end on the device — Tensor::create / copy / seblas::conv ... / seann::Conv2D, Linear — and checks results
// against the CPU oracle (linked here as the checker only). Mode "codec <dir>" writes, reads back and re-writes model
// files in <dir> for the Python test that checks their bytes against the file-format restatement. Mode "data <dir>" reads
// the dataset files the Python test put in <dir> through the seio data pipeline and leaves what it produced there; mode
// "train <dir>" trains a small classifier from a dataset file in <dir> with Sequential::train.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <random>
#include <stdexcept>
#include <vector>

#include "../../crusaderbackend_amd/csrc/crb_common.h"
#include "../../crusaderbackend_amd/host/seann/operands/Conv2D.h"
#include "../../crusaderbackend_amd/host/seann/containers/Sequential.h"
#include "../../crusaderbackend_amd/host/seann/operands/Elementwise.h"
#include "../../crusaderbackend_amd/host/seann/operands/Linear.h"
#include "../../crusaderbackend_amd/host/seann/operands/ShortcutEndpoint.h"
#include "../../crusaderbackend_amd/host/seio/data/Dataset.h"
#include "../../crusaderbackend_amd/host/seio/modelcache/codec.h"

extern "C" {
void oracle_sgemm(const float *, const float *, float *, uint32_t, uint32_t, uint32_t, uint32_t, int);
void oracle_sgemmNT(const float *, const float *, float *, uint32_t, uint32_t, uint32_t, int);
void oracle_linear(const float *, const float *, const float *, float *, uint32_t, uint32_t, uint32_t, int);
void oracle_linearXGrad(const float *, const float *, float *, uint32_t, uint32_t, uint32_t, int);
void oracle_linearParamGrad(const float *, const float *, float *, float *, uint32_t, uint32_t, uint32_t, int);
void oracle_conv(const float *, const float *, float *, const float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                 uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int);
void oracle_convDerive(const float *, const float *, float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                       uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int);
void oracle_convError(const float *, const float *, float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                      uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, int);
void oracle_relu(const float *, float *, uint32_t);
void oracle_reluGradFast(const float *, const float *, float *, uint32_t);
void oracle_maxPool(const float *, float *, float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t);
void oracle_maxPoolBack(float *, const float *, float *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t);
void oracle_softmax(const float *, float *, uint32_t, uint32_t);
void oracle_crossEntropyLoss(const float *, const float *, float *, uint32_t);
float oracle_crossEntropyCalc(const float *, const float *, uint32_t);
void oracle_momentumApply(float *, float *, float *, uint32_t, float, float, float);
void oracle_batchNorm(const float *, const float *, const float *, float *, float *, float *, float *, uint32_t, uint32_t);
void oracle_batchNormGrad(const float *, const float *, const float *, float *, uint32_t, uint32_t);
void oracle_batchNormParamGrads(const float *, const float *, float *, float *, uint32_t, uint32_t);
}

using namespace seblas;
static int g_fail = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
            ++g_fail;                                                        \
        }                                                                    \
    } while (0)

template <class F>
static bool throws_invalid(F f) {
    try {
        f();
    } catch (const std::invalid_argument &) {
        return true;
    } catch (...) {
        return false;
    }
    return false;
}

static void host_tests() {
    // shape constructor rules (Tensor.cuh:67-76)
    shape4 a(3, 5), b(2, 3, 5), c(7, 2, 3, 5);
    CHECK(a.n == 1 && a.c == 1 && a.h == 3 && a.w == 5 && a.size == 15);
    CHECK(b.n == 1 && b.c == 2 && b.h == 3 && b.w == 5 && b.size == 30);
    CHECK(c.n == 7 && c.size == 210);
    CHECK(c.toString() == "(7,2,3,5)");
    CHECK((index4(1, 2, 3, 4) + index4(1, 1, 1, 1)) == index4(2, 3, 4, 5));

    // exact division helper against the hardware divide
    std::mt19937 gen(7);
    const uint32_t divisors[] = {1, 2, 3, 5, 7, 9, 16, 17, 64, 144, 255, 256, 1000, 1024, 65535, 65536, 1u << 20, 0x7fffffffu, 0xffffffffu};
    for (uint32_t d : divisors) {
        crb::FastDiv fd(d);
        const uint32_t edge[] = {0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 0x7fffffffu, 0xfffffffeu, 0xffffffffu};
        for (uint32_t n : edge) CHECK(fd.div(n) == n / d);
        for (int i = 0; i < 20000; ++i) {
            uint32_t n = gen();
            uint32_t q, r;
            fd.divmod(n, q, r);
            CHECK(q == n / d && r == n % d);
        }
    }

    // descriptors can be declared, reshaped and attached without a device
    Tensor *t = Tensor::declare(2, 3, 4, 5);
    CHECK(t->dims.size == 120 && t->elements == nullptr);
    t->reshape(6, 20);
    CHECK(t->dims.h == 6 && t->dims.w == 20 && t->dims.n == 1);
    CHECK(throws_invalid([&] { t->reshape(7, 20); }));
    float backing[120];
    t->attach(backing, -1);
    CHECK(t->elements == backing && t->deviceId == -1);
    t->constFill(2.0f);
    Tensor *u = Tensor::declare(6, 20)->attach(backing, -1);
    *t + u;  // host branch of operator+: in-place add (aliasing itself doubles)
    CHECK(backing[0] == 4.0f && backing[119] == 4.0f);

    // shape violations are reported as std::invalid_argument before any device work
    Tensor *A = Tensor::declare(4, 6), *B = Tensor::declare(5, 8), *C = Tensor::declare(4, 8);
    CHECK(throws_invalid([&] { sgemm(A, B, C); }));       // A.w != B.h
    CHECK(throws_invalid([&] { sgemmNT(A, B, C); }));     // A.w != B.w
    CHECK(throws_invalid([&] { sgemmTN(A, B, C); }));
    Tensor *W = Tensor::declare(8, 3, 3, 3), *X = Tensor::declare(2, 3, 8, 8), *Y = Tensor::declare(2, 8, 7, 8);
    CHECK(throws_invalid([&] { conv(W, X, Y, 1, 1, 1, 1, nullptr); }));                      // rows relation
    Tensor *Y2 = Tensor::declare(2, 9, 8, 8);
    CHECK(throws_invalid([&] { conv(W, X, Y2, 1, 1, 1, 1, nullptr); }));                     // channels relation
    Tensor *Y3 = Tensor::declare(3, 8, 8, 8);
    CHECK(throws_invalid([&] { conv(W, X, Y3, 1, 1, 1, 1, nullptr); }));                     // batch relation
    Tensor *lx = Tensor::declare(4, 1, 10, 1), *lw = Tensor::declare(6, 11), *lb = Tensor::declare(6, 1), *ly = Tensor::declare(4, 1, 6, 1);
    CHECK(throws_invalid([&] { linear(lx, lw, lb, ly); }));                                  // W.w != X.h

    // operand shape inference (Conv2D.cuh:40-44, Linear.cu:9-13) is pure host arithmetic on declared shapes
    shape4 in(128, 16, 32, 32);
    uint32_t oh = (in.h + 2 * 1 - 3) / 2 + 1;
    CHECK(oh == 16);
}

static double tol(double ref, double rms, uint32_t K) { return 1e-5 * std::sqrt(double(K)) * std::fmax(std::fabs(ref), rms); }

static void compare(const char *what, const std::vector<float> &got, const std::vector<float> &ref, uint32_t K) {
    double ss = 0;
    for (float v : ref) ss += double(v) * v;
    double rms = std::sqrt(ss / double(ref.size()));
    size_t bad = 0;
    for (size_t i = 0; i < ref.size(); ++i)
        if (!(std::fabs(double(got[i]) - ref[i]) <= tol(ref[i], rms, K))) ++bad;
    if (bad) {
        std::printf("FAIL %s: %zu/%zu outside tolerance\n", what, bad, ref.size());
        ++g_fail;
    }
}

static std::vector<float> pull(Tensor *t) {
    std::vector<float> v(t->dims.size);
    Tensor *h = t->ripOffDevice();
    std::memcpy(v.data(), h->elements, sizeof(float) * v.size());
    h->eliminateHost();
    return v;
}

static Tensor *push(shape4 s, const std::vector<float> &v) {
    Tensor *h = Tensor::createHost(s);
    std::memcpy(h->elements, v.data(), sizeof(float) * v.size());
    return h->toDevice();
}

static std::vector<float> randn(size_t n, uint32_t seed, float sd = 1.0f) {
    std::mt19937 g(seed);
    std::normal_distribution<float> d(0.f, sd);
    std::vector<float> v(n);
    for (auto &x : v) x = d(g);
    return v;
}

static void gpu_tests() {
    // raw operator API: sgemm with a batched B, and sgemmNT
    {
        const uint32_t M = 70, K = 36, N = 52, batch = 3;
        auto a = randn(M * K, 1), b = randn(batch * K * N, 2);
        Tensor *A = push(shape4(M, K), a), *B = push(shape4(batch, 1, K, N), b), *C = Tensor::create(batch, 1, M, N);
        CHECK(sgemm(A, B, C) == C);
        std::vector<float> ref(batch * M * N);
        oracle_sgemm(a.data(), b.data(), ref.data(), M, N, K, batch, 4);
        compare("seblas::sgemm", pull(C), ref, K);
        A->eliminate(), B->eliminate(), C->eliminate();
    }
    // seann::Conv2D: forward, xGrads (with a non-zero reserve gradient folded in first), paramGrads
    for (int stride = 1; stride <= 2; ++stride) {
        const uint32_t N = 4, IC = 6, H = 12, OC = 10;
        seann::Conv2D op(shape4(OC, IC, 3, 3), stride, stride, 1, 1, true);
        op.initNetParams(nullptr, shape4(N, IC, H, H));
        seann::Parameter *src = seann::Parameter::create(N, IC, H, H);
        op.bindInput(src);
        op.randFillNetParams();
        const uint32_t OH = op.Y->A->dims.h;
        CHECK(OH == (H + 2 - 3) / stride + 1 && op.Y->A->dims.c == OC && op.Y->A->dims.n == N);
        auto x = randn(N * IC * H * H, 3), dy = randn(N * OC * OH * OH, 4), rs = randn(N * OC * OH * OH, 5);
        Tensor *hx = Tensor::createHost(src->A->dims);
        std::memcpy(hx->elements, x.data(), x.size() * 4);
        hx->copyToH2D(src->A);
        Tensor *hd = Tensor::createHost(op.Y->dA->dims);
        std::memcpy(hd->elements, dy.data(), dy.size() * 4);
        hd->copyToH2D(op.Y->dA);
        std::memcpy(hd->elements, rs.data(), rs.size() * 4);
        hd->copyToH2D(op.Y->dAReserve);
        auto w = pull(op.filter->data()), bv = pull(op.bias->data());

        op.forward();
        std::vector<float> ref(N * OC * OH * OH);
        oracle_conv(w.data(), x.data(), ref.data(), bv.data(), N, IC, H, H, OC, 3, 3, OH, OH, stride, stride, 1, 1, 4);
        compare("Conv2D::forward", pull(op.Y->A), ref, IC * 9);

        op.xGrads();  // dA += dAReserve; dX = dgrad(dA); reserve zeroed
        std::vector<float> dsum(dy.size());
        for (size_t i = 0; i < dy.size(); ++i) dsum[i] = dy[i] + rs[i];
        std::vector<float> refdx(x.size());
        oracle_convDerive(w.data(), dsum.data(), refdx.data(), N, IC, H, H, OC, 3, 3, OH, OH, stride, stride, 1, 1, 4);
        compare("Conv2D::xGrads", pull(src->dA), refdx, OC * 9);
        auto z = pull(op.Y->dAReserve);
        bool allzero = true;
        for (float v : z) allzero = allzero && v == 0.0f;
        CHECK(allzero);

        op.zeroGrads();
        op.paramGrads();
        std::vector<float> refdw(w.size(), 0.0f);
        oracle_convError(dsum.data(), x.data(), refdw.data(), N, IC, H, H, OC, 3, 3, OH, OH, stride, stride, 1, 1, 4);
        compare("Conv2D::paramGrads dW", pull(op.filter->grad()), refdw, N * OH * OH);
        std::vector<float> refdb(OC, 0.0f);
        for (uint32_t n = 0; n < N; ++n)
            for (uint32_t c = 0; c < OC; ++c)
                for (uint32_t i = 0; i < OH * OH; ++i) refdb[c] += dsum[(n * OC + c) * OH * OH + i];
        compare("Conv2D::paramGrads dB", pull(op.bias->grad()), refdb, N * OH * OH);
        // convError returns its first argument
        CHECK(convError(op.Y->dA, op.X->A, op.filter->grad(), stride, stride, 1, 1) == op.Y->dA);
    }
    // seann::Linear on a 4-D input (flattened to IN = c*h*w)
    {
        const uint32_t N = 9, OUT = 20;
        seann::Linear op(OUT);
        op.initNetParams(nullptr, shape4(N, 4, 3, 5));
        CHECK(op.INPUT_SIZE == 60 && op.X->A->dims.h == 60 && op.X->A->dims.w == 1);
        seann::Parameter *src = seann::Parameter::create(N, 4, 3, 5);
        op.bindInput(src);
        op.randFillNetParams();
        auto x = randn(N * 60, 6), dy = randn(N * OUT, 7);
        Tensor *hx = Tensor::createHost(src->A->dims);
        std::memcpy(hx->elements, x.data(), x.size() * 4);
        hx->copyToH2D(src->A);
        Tensor *hd = Tensor::createHost(op.Y->dA->dims);
        std::memcpy(hd->elements, dy.data(), dy.size() * 4);
        hd->copyToH2D(op.Y->dA);
        auto w = pull(op.weights->data()), b = pull(op.biases->data());
        op.forward();
        std::vector<float> ref(N * OUT), refdx(N * 60), refdw(OUT * 60, 0.f), refdb(OUT, 0.f);
        oracle_linear(x.data(), w.data(), b.data(), ref.data(), N, 60, OUT, 2);
        compare("Linear::forward", pull(op.Y->A), ref, 60);
        op.xGrads();
        oracle_linearXGrad(dy.data(), w.data(), refdx.data(), N, 60, OUT, 2);
        compare("Linear::xGrads", pull(src->dA), refdx, OUT);
        op.paramGrads();
        oracle_linearParamGrad(dy.data(), x.data(), refdw.data(), refdb.data(), N, 60, OUT, 2);
        compare("Linear::paramGrads dW", pull(op.weights->grad()), refdw, N);
        compare("Linear::paramGrads dB", pull(op.biases->grad()), refdb, N);
    }
}

// The elementwise / reduction operators through the seblas signatures: relu -> maxPool -> softmax -> cross-entropy and
// back, then a momentum step, each against the CPU oracle (bit-exact except where exp/log and summation order differ).
static void gpu_elementwise_tests() {
    const uint32_t N = 6, C = 5, H = 8, W = 8, n = N * C * H * W;
    auto x = randn(n, 21), dy = randn(n, 22);
    Tensor *X = push(shape4(N, C, H, W), x), *Y = Tensor::create(N, C, H, W), *dY = push(shape4(N, C, H, W), dy);
    Tensor *dX = Tensor::create(N, C, H, W);
    CHECK(relu(X, Y) == Y);
    std::vector<float> ry(n), rdx(n);
    oracle_relu(x.data(), ry.data(), n);
    CHECK(pull(Y) == ry);
    CHECK(reluGradFast(X, dY, dX) == dX);
    oracle_reluGradFast(x.data(), dy.data(), rdx.data(), n);
    CHECK(pull(dX) == rdx);

    // pooling: record has the MaxPool2D operand's shape (MaxPool2D.cuh:47-51)
    Tensor *P = Tensor::create(N, C, H / 2, W / 2), *rec = Tensor::create(N, C, H, W);
    maxPool(Y, P, rec, 2, 2, 2, 2);
    std::vector<float> rp(n / 4), rrec(n), rback(n);
    oracle_maxPool(ry.data(), rp.data(), rrec.data(), N * C, H, W, 2, 2);
    CHECK(pull(P) == rp);
    CHECK(pull(rec) == rrec);
    auto dp = randn(n / 4, 23);
    Tensor *dP = push(shape4(N, C, H / 2, W / 2), dp);
    maxPoolBack(dX, dP, rec, 2, 2, 2, 2);
    oracle_maxPoolBack(rback.data(), dp.data(), rrec.data(), N * C, H, W, 2, 2);
    CHECK(pull(dX) == rback);
    CHECK(pull(rec) == rrec);  // both cleared
    CHECK(throws_invalid([&] { maxPool(Y, P, rec, 2, 2, 3, 3); }));   // shape relationship (cuPool.cu:136-137)
    CHECK(throws_invalid([&] { maxPool(Y, Y, rec, 2, 2, 2, 2); }));

    // softmax over rows of 10, cross-entropy value and gradient
    const uint32_t rows = 16, classes = 10;
    auto z = randn(rows * classes, 24, 2.0f);
    std::vector<float> lab(rows * classes, 0.f);
    for (uint32_t r = 0; r < rows; ++r) lab[r * classes + (r * 7) % classes] = 1.f;
    seann::Parameter *S = seann::Parameter::create(rows, 1, classes, 1);
    Tensor *Z = push(shape4(rows, 1, classes, 1), z), *L = push(shape4(rows, 1, classes, 1), lab);
    CHECK(softmax(Z, S->A, nullptr, classes) == S->A);
    std::vector<float> rs(rows * classes), rg(rows * classes);
    oracle_softmax(z.data(), rs.data(), rows, classes);
    compare("seblas::softmax", pull(S->A), rs, 1);
    auto s_gpu = pull(S->A);
    crossEntropyLoss(S, L);
    oracle_crossEntropyLoss(s_gpu.data(), lab.data(), rg.data(), rows * classes);
    CHECK(pull(S->dA) == rg);
    Tensor *buf = Tensor::create(rows, 1, classes, 1);
    const float loss = crossEntropyCalc(S, L, buf), rloss = oracle_crossEntropyCalc(s_gpu.data(), lab.data(), rows * classes);
    CHECK(std::fabs(loss - rloss) <= 1e-5f * std::fabs(rloss) * std::sqrt(float(rows * classes)));
    CHECK(throws_invalid([&] { softmax(Z, S->A, nullptr, 7); }));  // cuReduce.cu:297

    // seann::BatchNorm: forward, xGrads, paramGrads (gamma's gradient lands in gamma, beta's in beta)
    {
        const uint32_t bn = 24, bc = 3, bh = 5, F = bc * bh * bh;
        seann::BatchNorm op;
        op.initNetParams(nullptr, shape4(bn, bc, bh, bh));
        seann::Parameter *src = seann::Parameter::create(bn, bc, bh, bh);
        op.bindInput(src);
        op.randFillNetParams();
        auto bx = randn(bn * F, 41, 2.0f), bdy = randn(bn * F, 42), bg = randn(F, 43), bb = randn(F, 44);
        for (auto &v : bg) v += 1.0f;
        push(src->A->dims, bx)->copyToD2D(src->A);
        push(op.gamma->data()->dims, bg)->copyToD2D(op.gamma->data());
        push(op.beta->data()->dims, bb)->copyToD2D(op.beta->data());
        push(op.Y->dA->dims, bdy)->copyToD2D(op.Y->dA);
        op.forward();
        std::vector<float> rY(bn * F), rxh(bn * F), rm(F), rv(F), rdx(bn * F), rdg(F), rdb(F);
        oracle_batchNorm(bx.data(), bb.data(), bg.data(), rm.data(), rv.data(), rY.data(), rxh.data(), bn, F);
        compare("BatchNorm::forward", pull(op.Y->A), rY, bn * 16);
        compare("BatchNorm mean", pull(op.mean), rm, bn * 16);
        op.xGrads();
        oracle_batchNormGrad(bdy.data(), bg.data(), bx.data(), rdx.data(), bn, F);
        compare("BatchNorm::xGrads", pull(src->dA), rdx, bn * 64);
        op.paramGrads();
        auto xh_gpu = pull(op.xHatP);
        oracle_batchNormParamGrads(bdy.data(), xh_gpu.data(), rdg.data(), rdb.data(), bn, F);
        compare("BatchNorm dGamma", pull(op.gamma->grad()), rdg, bn * 16);
        compare("BatchNorm dBeta", pull(op.beta->grad()), rdb, bn * 16);
        CHECK(throws_invalid([&] { batchNorm(src->A, op.beta->data(), op.gamma->data(), op.mean, op.variance, op.Y->A, op.mean); }));
    }

    // Tensor arithmetic used by the loss and the optimizer, then one momentum step with weight decay
    auto a = randn(1000, 25), b = randn(1000, 26), m = randn(1000, 27);
    Tensor *A = push(shape4(1000, 1), a), *B = push(shape4(1000, 1), b), *M = push(shape4(1000, 1), m);
    CHECK((*A - B) == A);
    auto ra = a;
    for (size_t i = 0; i < ra.size(); ++i) ra[i] = a[i] - b[i];
    CHECK(pull(A) == ra);
    CHECK((*A * 0.5f) == A);
    for (auto &v : ra) v *= 0.5f;
    CHECK(pull(A) == ra);
    auto rb = b, rm = m;
    momentumApplyDecay(A, B, M, 0.01f, 0.9f, 5e-4f);
    oracle_momentumApply(ra.data(), rb.data(), rm.data(), 1000, 0.01f, 0.9f, 1.0f - 5e-4f);
    CHECK(pull(A) == ra);
    CHECK(pull(M) == rm);
    CHECK(pull(B) == rb);  // gradient cleared
    momentumApply(A, B, M, 0.01f, 0.9f);
    oracle_momentumApply(ra.data(), rb.data(), rm.data(), 1000, 0.01f, 0.9f, 1.0f);
    CHECK(pull(A) == ra);
}

// seann::Sequential with residual connections (identity and projection shortcuts), the parameter-free operands and the
// momentum optimizer: one training step through the container, and the same step written out by hand with the seblas
// operators on separate tensors. Both run the same deterministic kernels, so every tensor must agree bit for bit; that
// pins the graph wiring (input aliasing, reserve gradients of the shortcuts, update order), not the arithmetic, which the
// operator tests pin. The forward result is also checked against the CPU oracle.
static Tensor *clone(Tensor *t) {
    Tensor *c = Tensor::create(t->dims);
    t->copyToD2D(c);
    return c;
}

static void gpu_sequential_tests() {
    using namespace seann;
    const uint32_t N = 4;
    auto *c1 = new Conv2D(shape4(8, 3, 3, 3), 1, 1, 1, 1, true);
    auto *c2 = new Conv2D(shape4(8, 8, 3, 3), 1, 1, 1, 1, true);
    auto *c3 = new Conv2D(shape4(8, 8, 3, 3), 1, 1, 1, 1, false);
    auto *c4 = new Conv2D(shape4(16, 8, 3, 3), 2, 2, 1, 1, true);
    auto *cp = new Conv2D(shape4(16, 8, 1, 1), 2, 2, 0, 0, false);  // projection shortcut
    auto *fc = new Linear(10);
    OPTIMIZER_MOMENTUM opt(0.05f, 0.9f);
    Sequential net(shape4(N, 3, 8, 8),
                   {c1, new ReLU(), new MaxPool2D(2, 2, 2, 2),
                    new ShortcutEndpoint(false, 1, {}), c2, new ReLU(), c3, new ShortcutEndpoint(true, 1, {}), new ReLU(),
                    new ShortcutEndpoint(false, 2, {}), c4, new ShortcutEndpoint(true, 2, {cp}), new ReLU(),
                    fc, new Softmax()});
    net.construct(&opt);
    net.setLoss(crossEntropyLoss, crossEntropyCalc);
    net.randInit();
    CHECK(net.netY->A->dims.size == N * 10);
    CHECK(c4->Y->A->dims == shape4(N, 16, 2, 2) && cp->Y->A->dims == shape4(N, 16, 2, 2));

    auto x = randn(N * 3 * 8 * 8, 31);
    std::vector<float> lab(N * 10, 0.f);
    for (uint32_t n = 0; n < N; ++n) lab[n * 10 + (3 * n + 1) % 10] = 1.f;
    Tensor *X = push(shape4(N, 3, 8, 8), x), *L = push(shape4(N, 1, 10, 1), lab);

    // copies of the initial parameters for the hand-written step
    Tensor *w1 = clone(c1->filter->data()), *b1 = clone(c1->bias->data()), *w2 = clone(c2->filter->data()),
           *b2 = clone(c2->bias->data()), *w3 = clone(c3->filter->data()), *w4 = clone(c4->filter->data()),
           *b4 = clone(c4->bias->data()), *wp = clone(cp->filter->data()), *wf = clone(fc->weights->data()),
           *bf = clone(fc->biases->data());

    net.forward(X);
    net.backward(L);
    Tensor *lossBuf = Tensor::create(net.netY->A->dims);
    const float loss = net.lossFW(net.netY, L, lossBuf);
    auto g_w1 = pull(c1->filter->grad()), g_b1 = pull(c1->bias->grad()), g_w3 = pull(c3->filter->grad()),
         g_wp = pull(cp->filter->grad()), g_wf = pull(fc->weights->grad()), g_dx = pull(net.netX->dA);
    auto probs = pull(net.netY->A);
    net.learn();

    // ---- the same step by hand ----
    auto T = [&](uint32_t c, uint32_t h) { return Tensor::create(N, c, h, h); };
    Tensor *z1 = T(8, 8), *a1 = T(8, 8), *p1 = T(8, 4), *rec = T(8, 8), *z2 = T(8, 4), *a2 = T(8, 4), *z3 = T(8, 4), *s1 = T(8, 4),
           *a3 = T(8, 4), *z4 = T(16, 2), *zp = T(16, 2), *s2 = T(16, 2), *a4 = T(16, 2);
    Tensor *zf = Tensor::create(N, 1, 10, 1);
    seblas::Parameter *P = seblas::Parameter::create(N, 1, 10, 1);
    conv(w1, X, z1, 1, 1, 1, 1, b1);
    relu(z1, a1);
    maxPool(a1, p1, rec, 2, 2, 2, 2);
    conv(w2, p1, z2, 1, 1, 1, 1, b2);
    relu(z2, a2);
    conv(w3, a2, z3, 1, 1, 1, 1, nullptr);
    z3->copyToD2D(s1);
    *s1 + p1;  // identity shortcut
    relu(s1, a3);
    conv(w4, a3, z4, 2, 2, 1, 1, b4);
    conv(wp, a3, zp, 2, 2, 0, 0, nullptr);
    z4->copyToD2D(s2);
    *s2 + zp;  // projection shortcut
    relu(s2, a4);
    Tensor *a4flat = Tensor::declare(N, 1, 64, 1)->attach(a4);
    linear(a4flat, wf, bf, zf);
    softmax(zf, P->A, nullptr, 10);
    CHECK(pull(P->A) == probs);
    {   // forward against the CPU oracle (first convolution + ReLU + pooling, then the final probabilities sum to 1)
        std::vector<float> rz(N * 8 * 64), ra(N * 8 * 64), rp(N * 8 * 16), rr(N * 8 * 64);
        auto hw1 = pull(w1), hb1 = pull(b1);
        oracle_conv(hw1.data(), x.data(), rz.data(), hb1.data(), N, 3, 8, 8, 8, 3, 3, 8, 8, 1, 1, 1, 1, 2);
        oracle_relu(rz.data(), ra.data(), N * 8 * 64);
        oracle_maxPool(ra.data(), rp.data(), rr.data(), N * 8, 8, 8, 2, 2);
        compare("Sequential: conv+relu+pool", pull(p1), rp, 27);
        for (uint32_t n = 0; n < N; ++n) {
            float sum = 0.f;
            for (int k = 0; k < 10; ++k) sum += probs[n * 10 + k];
            CHECK(std::fabs(sum - 1.f) < 1e-5f);
        }
    }
    crossEntropyLoss(P, L);
    CHECK(crossEntropyCalc(P, L, Tensor::create(N, 1, 10, 1)) == loss);
    // backward
    Tensor *dwf = Tensor::create(wf->dims), *dbf = Tensor::create(bf->dims), *da4 = Tensor::create(N, 1, 64, 1);
    linearXGrad(P->dA, wf, da4);
    linearParamGrad(P->dA, a4flat, dwf, dbf);
    CHECK(pull(dwf) == g_wf);
    Tensor *ds2 = T(16, 2), *da3 = T(8, 4), *da3p = T(8, 4), *dwp = Tensor::create(wp->dims), *dw4 = Tensor::create(w4->dims);
    reluGradFast(s2, Tensor::declare(N, 16, 2, 2)->attach(da4), ds2);
    convDerive(wp, ds2, da3p, 2, 2, 0, 0);  // projection branch
    convError(ds2, a3, dwp, 2, 2, 0, 0);
    CHECK(pull(dwp) == g_wp);
    convDerive(w4, ds2, da3, 2, 2, 1, 1);  // main branch
    convError(ds2, a3, dw4, 2, 2, 1, 1);
    *da3 + da3p;
    Tensor *ds1 = T(8, 4), *da2 = T(8, 4), *dz2 = T(8, 4), *dp1 = T(8, 4), *dw3 = Tensor::create(w3->dims), *dw2 = Tensor::create(w2->dims);
    reluGradFast(s1, da3, ds1);
    convDerive(w3, ds1, da2, 1, 1, 1, 1);
    convError(ds1, a2, dw3, 1, 1, 1, 1);
    CHECK(pull(dw3) == g_w3);
    reluGradFast(z2, da2, dz2);
    convDerive(w2, dz2, dp1, 1, 1, 1, 1);
    convError(dz2, p1, dw2, 1, 1, 1, 1);
    *dp1 + ds1;  // identity shortcut: the block input also receives the block output's gradient
    Tensor *da1 = T(8, 8), *dz1 = T(8, 8), *dx = Tensor::create(N, 3, 8, 8), *dw1 = Tensor::create(w1->dims), *db1 = Tensor::create(b1->dims);
    maxPoolBack(da1, dp1, rec, 2, 2, 2, 2);
    reluGradFast(z1, da1, dz1);
    convDerive(w1, dz1, dx, 1, 1, 1, 1);
    convError(dz1, X, dw1, 1, 1, 1, 1);
    CHECK(crb_conv_bias_grad(dz1->elements, db1->elements, N, 8, 64, nullptr) == 0);
    CHECK(pull(dw1) == g_w1);
    CHECK(pull(db1) == g_b1);
    CHECK(pull(dx) == g_dx);
    // update: weights decay with the optimizer's default L2, biases do not
    Tensor *m1 = Tensor::create(w1->dims), *mb1 = Tensor::create(b1->dims), *mf = Tensor::create(wf->dims);
    momentumApplyDecay(w1, dw1, m1, 0.05f, 0.9f, 0.0001f);
    momentumApplyDecay(b1, db1, mb1, 0.05f, 0.9f, 0.0f);
    momentumApplyDecay(wf, dwf, mf, 0.05f, 0.9f, 0.0001f);
    CHECK(pull(w1) == pull(c1->filter->data()));
    CHECK(pull(b1) == pull(c1->bias->data()));
    CHECK(pull(wf) == pull(fc->weights->data()));
    for (float v : pull(c1->filter->grad())) CHECK(v == 0.f);  // gradients are cleared by the step
    // a second forward after the update runs and changes the loss
    net.forward(X);
    CHECK(net.lossFW(net.netY, L, lossBuf) != loss);
    // the two optional shortcuts change nothing: prune the reserve folds, update all parameters in one launch
    {
        auto before_w = pull(c2->filter->data());
        net.forward(X);
        net.backward(L);
        auto g_plain = pull(c2->filter->grad()), dx_plain = pull(net.netX->dA), gp_plain = pull(cp->filter->grad());
        net.zeroGrads();
        net.streamline();
        net.forward(X);
        net.backward(L);
        CHECK(pull(c2->filter->grad()) == g_plain);
        CHECK(pull(cp->filter->grad()) == gp_plain);
        CHECK(pull(net.netX->dA) == dx_plain);
        // fused update against the per-parameter update on a copy of the state
        Tensor *wc = clone(c2->filter->data()), *gc = clone(c2->filter->grad());
        Tensor *mc = clone(static_cast<Momentum *>(c2->filter->opt)->m);
        momentumApplyDecay(wc, gc, mc, 0.05f, 0.9f, 0.0001f);
        net.learnFused();
        CHECK(pull(c2->filter->data()) == pull(wc));
        CHECK(pull(static_cast<Momentum *>(c2->filter->opt)->m) == pull(mc));
        for (float v : pull(fc->biases->grad())) CHECK(v == 0.f);
        CHECK(pull(c2->filter->data()) != before_w);
    }
    // a convolution whose two gradients run as one launch (16 -> 16 channels on 32 x 32, with bias): same numbers as the
    // two separate calls, gradient accumulation included
    {
        const uint32_t B = 8;
        auto run = [&](int mode, std::vector<float> &dx, std::vector<float> &dw, std::vector<float> &db) {
            const bool fused = mode >= 1, sliced = mode == 2;
            std::vector<seblas::SliceSumItem> items;
            auto *cv = new Conv2D(shape4(16, 16, 3, 3), 1, 1, 1, 1, true);
            cv->initNetParams(nullptr, shape4(B, 16, 32, 32));
            cv->randFillNetParams();
            cv->X->instantiate();  // stand-alone operand: it owns its input
            if (fused) cv->fuseGrads();
            if (sliced) {
                cv->deferSliceSum(items);
                CHECK(items.size() == 1 && items[0].n_slices > 1 && items[0].count == 16 * 16 * 9);
            }
            auto xin = randn(B * 16 * 32 * 32, 61), dy = randn(B * 16 * 32 * 32, 62), g0 = randn(16 * 16 * 9, 63);
            CHECK(hipMemcpy(cv->X->A->elements, xin.data(), xin.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
            CHECK(hipMemcpy(cv->filter->grad()->elements, g0.data(), g0.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
            cv->forward();
            CHECK(hipMemcpy(cv->Y->dA->elements, dy.data(), dy.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
            cv->xGrads();
            cv->paramGrads();
            if (sliced) {  // the filter gradient is still what it was until the slices are summed
                CHECK(pull(cv->filter->grad()) == g0);
                sumSlicesMulti(items.data(), uint32_t(items.size()));
            }
            dx = pull(cv->X->dA), dw = pull(cv->filter->grad()), db = pull(cv->bias->grad());
            if (fused) {  // paramGrads on its own still computes the filter gradient
                cv->paramGrads();
                CHECK(pull(cv->filter->grad()) != dw);
            }
        };
        std::vector<float> dx1, dw1, db1, dx2, dw2, db2, dx3, dw3, db3;
        run(0, dx1, dw1, db1);
        run(1, dx2, dw2, db2);
        run(2, dx3, dw3, db3);
        CHECK(dx1 == dx2 && dw1 == dw2 && db1 == db2);
        CHECK(dx1 == dx3 && dw1 == dw3 && db1 == db3);
    }
    // the non-blocking mode gives the same numbers
    setBlocking(false);
    net.forward(X);
    net.backward(L);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    setBlocking(true);
    CHECK(throws_invalid([&] { Sequential bad(shape4(1, 3, 8, 8), {new ShortcutEndpoint(true, 9, {})}); bad.construct(nullptr); }));
}

// ---- model files -------------------------------------------------------------------------------------------------------
static void dump(const std::string &path, const std::vector<float> &v) {
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    f.write(reinterpret_cast<const char *>(v.data()), std::streamsize(v.size() * sizeof(float)));
}

static std::vector<float> slurp(const std::string &path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    std::vector<float> v(size_t(f.tellg()) / sizeof(float));
    f.seekg(0);
    f.read(reinterpret_cast<char *>(v.data()), std::streamsize(v.size() * sizeof(float)));
    return v;
}

static bool file_exists(const std::string &path) { return bool(std::ifstream(path)); }

static std::vector<float> all_params(const seann::Sequential &net) {
    std::vector<seann::NetParam *> ps;
    for (auto *op : net.operands) op->collectNetParams(ps);
    std::vector<float> out;
    for (auto *p : ps) {
        auto v = pull(p->data());
        out.insert(out.end(), v.begin(), v.end());
    }
    return out;
}

// A network with every operand type the file format carries here: saved, loaded, and the loaded copy must compute and
// train exactly like the original. Files are left in `dir` for the byte-level check.
static void codec_tests(const std::string &dir) {
    using namespace seann;
    const uint32_t N = 4;
    auto build = [&] {
        return new Sequential(shape4(N, 3, 8, 8),
                              {new Conv2D(shape4(8, 3, 3, 3), 1, 1, 1, 1, true), new BatchNorm(), new ReLU(), new MaxPool2D(2, 2, 2, 2),
                               new ShortcutEndpoint(false, 1, {}), new Conv2D(shape4(8, 8, 3, 3), 1, 1, 1, 1, false), new BatchNorm(),
                               new ShortcutEndpoint(true, 1, {}), new ReLU(),
                               new ShortcutEndpoint(false, 2, {}), new Conv2D(shape4(16, 8, 3, 3), 2, 2, 1, 1, true),
                               new ShortcutEndpoint(true, 2, {new Conv2D(shape4(16, 8, 1, 1), 2, 2, 0, 0, false), new BatchNorm()}),
                               new ReLU(), new Linear(10), new Softmax()});
    };
    OPTIMIZER_MOMENTUM opt(0.05f, 0.9f);
    Sequential *net = build();
    net->construct(&opt);
    net->setLoss(crossEntropyLoss, crossEntropyCalc);
    net->randInit();
    {  // batch-norm parameters away from their 0 / 1 start so that their order in the file matters
        std::vector<NetParam *> ps;
        for (auto *op : net->operands) op->collectNetParams(ps);
        uint32_t seed = 900;
        for (auto *op : net->operands) {
            auto give = [&](BatchNorm *bn) {
                auto b = randn(bn->beta->data()->dims.size, seed++, 0.3f), g = randn(bn->gamma->data()->dims.size, seed++, 0.2f);
                for (auto &v : g) v += 1.0f;
                CHECK(hipMemcpy(bn->beta->data()->elements, b.data(), b.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
                CHECK(hipMemcpy(bn->gamma->data()->elements, g.data(), g.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
            };
            if (auto *bn = dynamic_cast<BatchNorm *>(op)) give(bn);
            if (auto *se = dynamic_cast<ShortcutEndpoint *>(op))
                for (auto *b : se->branchOperands)
                    if (auto *bn = dynamic_cast<BatchNorm *>(b)) give(bn);
        }
    }
    auto x = randn(N * 3 * 8 * 8, 77);
    std::vector<float> lab(N * 10, 0.f);
    for (uint32_t n = 0; n < N; ++n) lab[n * 10 + (7 * n + 2) % 10] = 1.f;
    Tensor *X = push(shape4(N, 3, 8, 8), x), *L = push(shape4(N, 1, 10, 1), lab);

    const std::string fa = dir + "/a.crseq";
    seio::saveSequence(fa.c_str(), net, 17);
    dump(dir + "/a.params.f32", all_params(*net));
    auto y1 = pull(net->forward(X));
    dump(dir + "/a.x.f32", x);
    dump(dir + "/a.y.f32", y1);

    CHECK(seio::loadedEpochID(fa.c_str()) == 17);
    Sequential *twin = seio::loadSequence(fa.c_str(), shape4(N, 3, 8, 8), &opt);
    twin->setLoss(crossEntropyLoss, crossEntropyCalc);
    CHECK(twin->OPERAND_COUNT == net->OPERAND_COUNT);
    CHECK(all_params(*twin) == all_params(*net));
    auto y2 = pull(twin->forward(X));
    CHECK(y1 == y2);  // same kernels on the same values: identical bits
    // one training step on both: the loaded network is wired for backward and update as well
    net->backward(L), net->learn();
    twin->forward(X), twin->backward(L), twin->learn();
    CHECK(all_params(*twin) == all_params(*net));
    CHECK(pull(net->forward(X)) == pull(twin->forward(X)));
    // the streamlined form of the loaded network (one-launch convolution gradients, slices summed once, ReLUs absorbed by
    // the batch normalisation / closing endpoint before them, one-launch update) computes the same bits as the plain one
    {
        auto all_grads = [](const Sequential &n) {
            std::vector<NetParam *> ps;
            for (auto *op : n.operands) op->collectNetParams(ps);
            std::vector<float> out;
            for (auto *p : ps) {
                auto v = pull(p->grad());
                out.insert(out.end(), v.begin(), v.end());
            }
            return out;
        };
        twin->streamline();
        uint32_t absorbed = 0;
        for (auto *op : twin->operands)
            if (auto *r = dynamic_cast<ReLU *>(op)) absorbed += r->absorbedBy ? 1 : 0;
        CHECK(absorbed == 3);
        for (int step = 0; step < 2; step++) {
            CHECK(pull(net->forward(X)) == pull(twin->forward(X)));
            net->backward(L), twin->backward(L);
            CHECK(all_grads(*net) == all_grads(*twin));
            CHECK(pull(net->netX->dA) == pull(twin->netX->dA));
            net->learn(), twin->learnFused();
            CHECK(all_params(*net) == all_params(*twin));
        }
    }
    // a second save of an unchanged network replaces the file with the same bytes
    const std::string fa2 = dir + "/a2.crseq";
    seio::saveSequence(fa2.c_str(), twin, 18);
    seio::saveSequence(fa2.c_str(), twin, 18);
    dump(dir + "/a2.params.f32", all_params(*twin));

    // a file written by the format restatement: load, run, write again
    const std::string fb = dir + "/b.crseq";
    if (file_exists(fb)) {
        auto shp = slurp(dir + "/b.shape.f32");  // n, c, h, w
        shape4 in = shape4((uint32_t)shp[0], (uint32_t)shp[1], (uint32_t)shp[2], (uint32_t)shp[3]);
        Sequential *b = seio::loadSequence(fb.c_str(), in, nullptr);
        Tensor *BX = push(in, slurp(dir + "/b.x.f32"));
        dump(dir + "/b.y.f32", pull(b->forward(BX)));
        seio::saveSequence((dir + "/b2.crseq").c_str(), b, seio::loadedEpochID(fb.c_str()));
    }

    // malformed files are reported, not followed
    auto throws_runtime = [&](const std::string &path) {
        try {
            seio::loadSequence(path.c_str(), shape4(N, 3, 8, 8), nullptr);
        } catch (const std::runtime_error &) {
            return true;
        } catch (...) {
            return false;
        }
        return false;
    };
    CHECK(throws_runtime(dir + "/does_not_exist.crseq"));
    {
        std::ifstream src(fa, std::ios::binary);
        std::vector<char> bytes((std::istreambuf_iterator<char>(src)), std::istreambuf_iterator<char>());
        std::ofstream(dir + "/truncated.crseq", std::ios::binary).write(bytes.data(), std::streamsize(bytes.size() - 40));
        bytes[0] ^= 1;
        std::ofstream(dir + "/badmagic.crseq", std::ios::binary).write(bytes.data(), std::streamsize(bytes.size()));
    }
    CHECK(throws_runtime(dir + "/truncated.crseq"));
    CHECK(throws_runtime(dir + "/badmagic.crseq"));
}

// ---- data pipeline ---------------------------------------------------------------------------------------------------------
template <class T>
static std::vector<T> slurp_as(const std::string &path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    std::vector<T> v(size_t(f.tellg()) / sizeof(T));
    f.seekg(0);
    f.read(reinterpret_cast<char *>(v.data()), std::streamsize(v.size() * sizeof(T)));
    return v;
}
template <class T>
static void dump_as(const std::string &path, const std::vector<T> &v) {
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    f.write(reinterpret_cast<const char *>(v.data()), std::streamsize(v.size() * sizeof(T)));
}

// draws come from a file, so that the Python side knows which records a batch holds
struct ScriptedFetcher : public seio::DataFetcher {
    std::vector<uint32_t> draws, taken;
    size_t at = 0;
    using seio::DataFetcher::DataFetcher;
    uint32_t draw(uint32_t remaining) override {
        uint32_t d = draws.at(at++) % remaining;
        taken.push_back(d);
        return d;
    }
};

static void data_tests(const std::string &dir) {
    using namespace seio;
    // dataset of 20 records (3 x 8 x 8 pixels, 10 label values): 16 per epoch + 4 held out
    const shape4 dataShape(3, 8, 8), labelShape(10, 1);
    auto *loader = new CrdatLoader();
    auto *fetcher = new ScriptedFetcher(dir, "set", 16, 4, loader, 1);
    fetcher->draws = slurp_as<uint32_t>(dir + "/draws.u32");

    // the reference's form of a record: host tensors of floats
    Tensor *hx = Tensor::createHost(dataShape), *hl = Tensor::createHost(labelShape);
    loader->loadData(hx, hl, dir.c_str(), "set", 7);
    dump(dir + "/rec7.x.f32", std::vector<float>(hx->elements, hx->elements + hx->dims.size));
    dump(dir + "/rec7.label.f32", std::vector<float>(hl->elements, hl->elements + hl->dims.size));
    bool past_end = false;
    try {
        loader->loadData(hx, hl, dir.c_str(), "set", 20);
    } catch (const std::out_of_range &) {
        past_end = true;
    }
    CHECK(past_end);

    Dataset *set = Dataset::construct(8, 4, 16, 10, dataShape, labelShape, 5);
    set->setDataFetcher(fetcher);
    set->setProcSteps({new UniformNorm()});
    set->setAugmentSteps({new RandFlipW(4, dataShape, labelShape), new RandCorp(4, dataShape, labelShape, 2, 2)});
    std::vector<uint32_t> order;
    for (int b = 0; b < 3; b++) {
        const size_t before = fetcher->taken.size();
        if (b == 1)
            set->genBatchAsync().join();
        else
            set->genBatch();
        CHECK(fetcher->taken.size() == before + 8);
        CHECK(set->batchID == uint32_t(b + 1) && set->epochID == uint32_t((b + 1) * 8 / 16));
        std::vector<float> x, lab;
        for (uint32_t i = 0; i < 2; i++) {
            Data *mb = set->dataBatch[b % 2][i];
            CHECK(mb->X->dims == shape4(4, 3, 8, 8) && mb->label->dims == shape4(4, 1, 10, 1));
            auto vx = pull(mb->X), vl = pull(mb->label);
            x.insert(x.end(), vx.begin(), vx.end());
            lab.insert(lab.end(), vl.begin(), vl.end());
        }
        dump(dir + "/batch" + std::to_string(b) + ".x.f32", x);
        dump(dir + "/batch" + std::to_string(b) + ".label.f32", lab);
        std::vector<int32_t> aug;
        for (const ImageAug &a : set->lastAugmentations()) aug.push_back(a.dh), aug.push_back(a.dw), aug.push_back(int32_t(a.flags));
        dump_as(dir + "/batch" + std::to_string(b) + ".aug.i32", aug);
    }
    dump_as(dir + "/taken.u32", fetcher->taken);

    // a second dataset without transform or augmentation, distribution scaling on a third; seeded random sampling
    auto *plain = Dataset::construct(4, 2, 16, 1, dataShape, labelShape, 3);
    auto *f2 = new ScriptedFetcher(dir, "set", 16, 4, new CrdatLoader(), 1);
    f2->draws = {3, 3, 0, 0};
    plain->setDataFetcher(f2);
    plain->genBatch();
    {
        std::vector<float> x;
        for (uint32_t i = 0; i < 2; i++) {
            auto v = pull(plain->dataBatch[0][i]->X);
            x.insert(x.end(), v.begin(), v.end());
        }
        dump(dir + "/plain.x.f32", x);
    }
    auto *dist = Dataset::construct(4, 4, 16, 1, dataShape, labelShape, 3);
    auto *f3 = new ScriptedFetcher(dir, "set", 16, 4, new CrdatLoader(), 1);
    f3->draws = {19, 0, 5, 5};
    dist->setDataFetcher(f3);
    dist->setProcSteps({new DistribNorm(0.5f, 0.25f)});
    dist->genBatch();
    dump(dir + "/dist.x.f32", pull(dist->dataBatch[0][0]->X));

    // sampling without replacement with the built-in generator: the first 20 fetches visit every record once
    DataFetcher rnd(dir, "set", 16, 4, new CrdatLoader(), 77);
    std::vector<int> seen(20, 0);
    for (int i = 0; i < 20; i++) seen[rnd.nextRecord()]++;
    bool once = true;
    for (int c : seen) once = once && c == 1;
    CHECK(once && rnd.remainedData == 16);
    std::vector<int> seen2(20, 0);
    for (int i = 0; i < 16; i++) seen2[rnd.nextRecord()]++;
    bool atmost = true;
    for (int c : seen2) atmost = atmost && c <= 1;
    CHECK(atmost);

    // CIFAR-10 binary batches: two files of 6 records
    CifarBinLoader cifar({dir + "/cifar_1.bin", dir + "/cifar_2.bin"}, 6);
    Tensor *cx = Tensor::createHost(shape4(3, 32, 32)), *cl = Tensor::createHost(shape4(10, 1));
    std::vector<float> cxs, cls;
    for (uint32_t id : {0u, 5u, 6u, 11u, 3u}) {
        cifar.loadData(cx, cl, "", "", id);
        cxs.insert(cxs.end(), cx->elements, cx->elements + 3072);
        cls.insert(cls.end(), cl->elements, cl->elements + 10);
    }
    dump(dir + "/cifar.x.f32", cxs);
    dump(dir + "/cifar.label.f32", cls);
    bool past = false;
    try {
        cifar.loadData(cx, cl, "", "", 12);
    } catch (const std::out_of_range &) {
        past = true;
    }
    CHECK(past);

    // argument checks
    CHECK(throws_invalid([&] { Dataset::construct(8, 3, 16, 1, dataShape, labelShape); }));
    CHECK(throws_invalid([&] { Dataset::construct(32, 4, 16, 1, dataShape, labelShape); }));
    CHECK(throws_invalid([&] { plain->setProcSteps({new UniformNorm(), new DistribNorm()}); }));
}

// ---- training loop -----------------------------------------------------------------------------------------------------------
static std::vector<float> g_train_loss, g_test_loss;
static void on_batch(uint32_t, uint32_t, float trainLoss, float testLoss) {
    g_train_loss.push_back(trainLoss);
    g_test_loss.push_back(testLoss);
}

// A small classifier trained from a .crdat file the Python test wrote (two classes, told apart by which half of the image
// is bright): the loss falls, the log and the epoch-0 model file appear, and the saved model loads.
static void train_tests(const std::string &dir) {
    using namespace seann;
    using namespace seio;
    const shape4 dataShape(1, 8, 8), labelShape(2, 1);
    const uint32_t MB = 8;
    Dataset *set = Dataset::construct(32, MB, 96, 3, dataShape, labelShape, 11);
    set->setDataFetcher(new DataFetcher(dir, "toy", 96, 16, new CrdatLoader(), 12));
    set->setProcSteps({new UniformNorm()});
    set->setAugmentSteps({new RandFlipW(MB, dataShape, labelShape)});  // would swap the classes if labels did not tell; kept off below
    set->setAugmentSteps({});
    set->allocTestSet();
    CHECK(set->TEST_SIZE == 16 && set->testset[1]->X->dims == shape4(MB, 1, 8, 8));

    OPTIMIZER_MOMENTUM opt(0.02f, 0.9f);
    Sequential net(shape4(MB, 1, 8, 8), {new Conv2D(shape4(4, 1, 3, 3), 1, 1, 1, 1, true), new ReLU(), new MaxPool2D(2, 2, 2, 2),
                                        new Linear(2), new Softmax()});
    net.construct(&opt);
    net.setLoss(crossEntropyLoss, crossEntropyCalc);
    net.randInit();
    CHECK(throws_invalid([&] { Sequential other(shape4(4, 1, 8, 8), {new Linear(2), new Softmax()}); other.construct(&opt);
                               other.setLoss(crossEntropyLoss, crossEntropyCalc); other.train(set, false, 1, dir.c_str()); }));
    net.train(set, true, 1, dir.c_str(), on_batch);
    // 3 epochs of 96 samples in batches of 32 are 9 batches; the epoch counter follows the batches formed, which run one
    // ahead of the batches trained on, so the loop (as in the reference) ends after training on 8
    CHECK(g_train_loss.size() == 8 && set->epochID == 3);
    if (g_train_loss.size() != 8) return;
    float first = (g_train_loss[0] + g_train_loss[1]) / 2, last = (g_train_loss[6] + g_train_loss[7]) / 2;
    std::printf("train loss %.4f -> %.4f, test loss %.4f -> %.4f\n", first, last, g_test_loss.front(), g_test_loss.back());
    CHECK(last < 0.7f * first);
    CHECK(g_test_loss.back() < g_test_loss.front());
    CHECK(file_exists(dir + "/cache.log") && file_exists(dir + "/cache.crseq"));
    CHECK(seio::loadedEpochID((dir + "/cache.crseq").c_str()) == 0);
    Sequential *back = seio::loadSequence((dir + "/cache.crseq").c_str(), shape4(MB, 1, 8, 8), nullptr);
    CHECK(back->OPERAND_COUNT == 5);
}

int main(int argc, char **argv) {
    const bool gpu = argc > 1 && std::strcmp(argv[1], "gpu") == 0;
    const bool codec = argc > 2 && std::strcmp(argv[1], "codec") == 0;
    try {
        if (codec) {
            setBlocking(true);
            codec_tests(argv[2]);
            std::printf("codec: %s\n", g_fail ? "FAILED" : "OK");
            return g_fail ? 1 : 0;
        }
        if (argc > 2 && std::strcmp(argv[1], "train") == 0) {
            setBlocking(true);
            train_tests(argv[2]);
            std::printf("train: %s\n", g_fail ? "FAILED" : "OK");
            return g_fail ? 1 : 0;
        }
        if (argc > 2 && std::strcmp(argv[1], "data") == 0) {
            setBlocking(true);
            data_tests(argv[2]);
            std::printf("data: %s\n", g_fail ? "FAILED" : "OK");
            return g_fail ? 1 : 0;
        }
        if (gpu) {
            gpu_tests();
            gpu_elementwise_tests();
            gpu_sequential_tests();
        }
        else
            host_tests();
    } catch (const std::exception &e) {
        std::printf("FAIL: unexpected exception: %s\n", e.what());
        return 2;
    }
    std::printf("%s: %s\n", gpu ? "gpu" : "host", g_fail ? "FAILED" : "OK");
    return g_fail ? 1 : 0;
}
