// seblas::Tensor for the HIP build: the same 4-D NCHW fp32 descriptor, ownership rules and method names as
// the reference (seblas/tensor/Tensor.cuh:48-208, Tensor.cu:353-460), minus the cuDNN descriptor field.
// Element (n,c,h,w) lives at ((n*C + c)*H + h)*W + w. deviceId: -1 host, 0 GPU.
// Tensors are created with declare()/create() and released with eliminate(); there is no RAII and ops
// never allocate or free — exactly the reference's contract.
#pragma once
#include <cstdint>
#include <string>
#include <utility>

namespace seblas {
typedef uint32_t uint32;
typedef uint64_t uint64;

struct index4 {
    uint32 n = 0, c = 0, h = 0, w = 0;
    index4() = default;
    index4(uint32 n, uint32 c, uint32 h, uint32 w) : n(n), c(c), h(h), w(w) {}
    index4(uint32 c, uint32 h, uint32 w) : c(c), h(h), w(w) {}
    index4(uint32 h, uint32 w) : h(h), w(w) {}
    index4 operator+(index4 o) const { return {n + o.n, c + o.c, h + o.h, w + o.w}; }
    index4 operator-(index4 o) const { return {n - o.n, c - o.c, h - o.h, w - o.w}; }
    bool operator==(index4 o) const { return n == o.n && c == o.c && h == o.h && w == o.w; }
    bool operator>(index4 o) const { return n > o.n && c > o.c && h > o.h && w > o.w; }
    bool operator<(index4 o) const { return n < o.n && c < o.c && h < o.h && w < o.w; }
    std::string toString() const {
        return "(" + std::to_string(n) + "," + std::to_string(c) + "," + std::to_string(h) + "," + std::to_string(w) + ")";
    }
};

// Two-argument form is a matrix (1,1,h,w); three-argument form is (1,c,h,w) (Tensor.cuh:67-76).
struct shape4 : public index4 {
    uint32 size = 0;
    shape4() = default;
    shape4(uint32 n, uint32 c, uint32 h, uint32 w) : index4(n, c, h, w) { size = n * c * h * w; }
    shape4(uint32 c, uint32 h, uint32 w) : index4(1, c, h, w) { size = c * h * w; }
    shape4(uint32 h, uint32 w) : index4(1, 1, h, w) { size = h * w; }
};

class Tensor {
public:
    shape4 dims;
    float *elements = nullptr;
    int deviceId = 0;

    static Tensor *declare(shape4 dims);
    template <typename... Args>
    static Tensor *declare(Args &&...args) { return declare(shape4(std::forward<Args>(args)...)); }
    static Tensor *create(shape4 dims) { return declare(dims)->instantiate(); }
    template <typename... Args>
    static Tensor *create(Args &&...args) { return create(shape4(std::forward<Args>(args)...)); }
    static Tensor *createHost(shape4 dims) { return declare(dims)->instantiateHost(); }
    template <typename... Args>
    static Tensor *createHost(Args... args) { return createHost(shape4(args...)); }

    Tensor *reshape(shape4 dim);  // requires equal element count
    template <typename... Args>
    Tensor *reshape(Args &&...args) { return reshape(shape4(std::forward<Args>(args)...)); }

    Tensor *instantiate();      // device buffer, zero-filled
    Tensor *destroy();
    void eliminate();           // destroy() + free the descriptor
    Tensor *instantiateHost();  // pinned host buffer
    Tensor *destroyHost();
    void eliminateHost();

    Tensor *toDevice();  // migrates; `this` is released
    Tensor *toHost();
    Tensor *ripOffDevice() const;  // host copy of a device tensor
    Tensor *ripOffHost() const;    // device copy of a host tensor

    Tensor *copyToH2D(Tensor *onDevice) const;
    Tensor *copyToD2H(Tensor *onHost) const;
    Tensor *copyToD2D(Tensor *onDevice) const;
    Tensor *copyToH2H(Tensor *onHost) const;

    Tensor *attach(Tensor *other);  // share other's storage (requires size <= other's)
    Tensor *attach(float *element, int deviceID);

    // The two elementwise members the conv/linear operands use on the path (Tensor.cu:118-132,294-304,
    // 462-483,638-657): in-place `*this += *other`, and fill. Device tensors run on the GPU.
    Tensor *operator+(Tensor *other);
    Tensor *constFill(float val);
    // `*this += *other; *other = 0` in one pass: what every operand's xGrads does with its reserve gradient
    // (`*Y->dA + Y->dAReserve` ... `Y->dAReserve->constFill(0)`, e.g. seann/operands/seblas/Conv2D.cu:19,21).
    Tensor *addAndClear(Tensor *other);
    // `*this -= *other` (Tensor.cu:485-506: the loss gradient) and `*this *= factor` (Tensor.cu:596-617: weight decay)
    Tensor *operator-(Tensor *other);
    Tensor *operator*(float factor);
    // Host-generated N(mean, stddev) from a fixed-seed mt19937 (the reference's wall-clock-seeded cuRAND
    // stream, Tensor.cu:306-322,667-683, is deliberately not reproduced).
    Tensor *randNormal(float mean, float stddev, uint32 seed = 0x5eb1a5u);
    Tensor *randUniform(float min, float max, uint32 seed = 0x5eb1a5u);

    float get(uint32 offset) const;
};
// The reference blocks the host after every operator and every device copy (cudaDeviceSynchronize / cudaMemcpy), and so
// does this layer by default. A caller that issues a whole step on the default stream and synchronises once can switch
// that off; device errors then surface at its own synchronisation point. No counterpart in the reference.
void setBlocking(bool blocking);
bool isBlocking();
}  // namespace seblas
