// seblas::Tensor / Parameter storage management on HIP (see Tensor.h for the contract being mirrored).
#include "Tensor.h"

#include <hip/hip_runtime_api.h>

#include <cstring>
#include <random>
#include <stdexcept>
#include <vector>

#include "../../../../include/crusader_hip.h"
#include "../assist/HipAssert.h"
#include "Parameter.h"

namespace seblas {

static void require(bool ok, const char *what) {
    if (!ok) throw std::invalid_argument(what);
}

void assertHip(const char *file, int line) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        throw std::runtime_error("line: " + std::to_string(line) + " file: " + file + " (" + hipGetErrorString(e) + ")");
}

void throwOnStatus(int status, const char *file, int line) {
    if (status == CRB_OK) return;
    std::string msg = std::string(crb_last_error_string()) + " [line: " + std::to_string(line) + " file: " + file + "]";
    if (status == CRB_EINVAL_SHAPE || status == CRB_ENULL) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

// Descriptors live in pinned host memory in the reference (cudaMallocHost, Tensor.cuh:97-106) because its
// kernels dereference them; here kernels take dimensions by value, so the descriptor is ordinary heap memory.
Tensor *Tensor::declare(shape4 dims) {
    Tensor *t = new Tensor();
    t->dims = dims;
    return t;
}

Tensor *Tensor::reshape(shape4 dim) {
    require(dim.size == dims.size, "Tensor::reshape: element counts differ");
    dims = dim;
    return this;
}

Tensor *Tensor::instantiate() {
    if (hipMalloc(reinterpret_cast<void **>(&elements), sizeof(float) * size_t(dims.size)) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    if (hipMemset(elements, 0, sizeof(float) * size_t(dims.size)) != hipSuccess) assertHip(__FILE__, __LINE__);
    deviceId = 0;
    return this;
}

Tensor *Tensor::destroy() {
    if (hipFree(elements) != hipSuccess) assertHip(__FILE__, __LINE__);
    elements = nullptr;
    return this;
}

void Tensor::eliminate() {
    destroy();
    delete this;
}

Tensor *Tensor::instantiateHost() {
    if (hipHostMalloc(reinterpret_cast<void **>(&elements), sizeof(float) * size_t(dims.size), hipHostMallocDefault) !=
        hipSuccess)
        assertHip(__FILE__, __LINE__);
    deviceId = -1;
    return this;
}

Tensor *Tensor::destroyHost() {
    if (hipHostFree(elements) != hipSuccess) assertHip(__FILE__, __LINE__);
    elements = nullptr;
    return this;
}

void Tensor::eliminateHost() {
    destroyHost();
    delete this;
}

Tensor *Tensor::toDevice() {
    Tensor *out = Tensor::declare(dims)->instantiate();
    copyToH2D(out);
    eliminateHost();
    return out;
}

Tensor *Tensor::toHost() {
    Tensor *out = Tensor::declare(dims)->instantiateHost();
    copyToD2H(out);
    eliminate();
    return out;
}

Tensor *Tensor::ripOffDevice() const {
    Tensor *out = Tensor::declare(dims)->instantiateHost();
    copyToD2H(out);
    return out;
}

Tensor *Tensor::ripOffHost() const {
    Tensor *out = Tensor::declare(dims)->instantiate();
    copyToH2D(out);
    return out;
}

static Tensor *copy(const Tensor *src, Tensor *dst, hipMemcpyKind kind) {
    require(src->dims.size == dst->dims.size, "Tensor::copyTo: element counts differ");
    if (hipMemcpy(dst->elements, src->elements, sizeof(float) * size_t(src->dims.size), kind) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    return dst;
}
Tensor *Tensor::copyToH2D(Tensor *onDevice) const { return copy(this, onDevice, hipMemcpyHostToDevice); }
Tensor *Tensor::copyToD2H(Tensor *onHost) const { return copy(this, onHost, hipMemcpyDeviceToHost); }
Tensor *Tensor::copyToD2D(Tensor *onDevice) const {  // a kernel on the default stream, so the host need not stall
    require(dims.size == onDevice->dims.size, "Tensor::copyToD2D: element counts differ");
    throwOnStatus(crb_tensor_copy(onDevice->elements, elements, dims.size, nullptr), __FILE__, __LINE__);
    if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(__FILE__, __LINE__);
    return onDevice;
}
Tensor *Tensor::copyToH2H(Tensor *onHost) const { return copy(this, onHost, hipMemcpyHostToHost); }

Tensor *Tensor::attach(Tensor *other) {
    require(dims.size <= other->dims.size, "Tensor::attach: target is smaller than this tensor");
    elements = other->elements;
    deviceId = other->deviceId;
    return this;
}

Tensor *Tensor::attach(float *element, int deviceID) {
    elements = element;
    deviceId = deviceID;
    return this;
}

static bool g_blocking = true;
void setBlocking(bool blocking) { g_blocking = blocking; }
bool isBlocking() { return g_blocking; }

// Every device operator ends like the reference's (cudaDeviceSynchronize(); assertCuda(...), e.g. Tensor.cu:482-483): status
// check, then — in blocking mode — a wait for the stream, so that an asynchronous fault surfaces at the operator that caused it.
static void launched(int status, const char *file, int line) {
    throwOnStatus(status, file, line);
    if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(file, line);
    assertHip(file, line);
}

Tensor *Tensor::operator+(Tensor *other) {
    require(dims.size == other->dims.size, "Tensor::operator+: element counts differ");
    require(deviceId == other->deviceId, "Tensor::operator+: tensors live on different devices");
    if (deviceId == -1) {
        for (uint32 i = 0; i < dims.size; ++i) elements[i] += other->elements[i];
        return this;
    }
    launched(crb_tensor_add_inplace(elements, other->elements, dims.size, nullptr), __FILE__, __LINE__);
    return this;
}

Tensor *Tensor::addAndClear(Tensor *other) {
    require(dims.size == other->dims.size, "Tensor::addAndClear: element counts differ");
    require(deviceId == other->deviceId, "Tensor::addAndClear: tensors live on different devices");
    if (deviceId == -1) {
        for (uint32 i = 0; i < dims.size; ++i) elements[i] += other->elements[i], other->elements[i] = 0.f;
        return this;
    }
    launched(crb_tensor_add_clear(elements, other->elements, dims.size, nullptr), __FILE__, __LINE__);
    return this;
}

Tensor *Tensor::operator-(Tensor *other) {
    require(dims.size == other->dims.size, "Tensor::operator-: element counts differ");
    require(deviceId == other->deviceId, "Tensor::operator-: tensors live on different devices");
    if (deviceId == -1) {
        for (uint32 i = 0; i < dims.size; ++i) elements[i] -= other->elements[i];
        return this;
    }
    launched(crb_tensor_sub_inplace(elements, other->elements, dims.size, nullptr), __FILE__, __LINE__);
    return this;
}

Tensor *Tensor::operator*(float factor) {
    if (deviceId == -1) {
        for (uint32 i = 0; i < dims.size; ++i) elements[i] *= factor;
        return this;
    }
    launched(crb_tensor_scale_inplace(elements, factor, dims.size, nullptr), __FILE__, __LINE__);
    return this;
}

Tensor *Tensor::constFill(float val) {
    if (deviceId == -1) {
        for (uint32 i = 0; i < dims.size; ++i) elements[i] = val;
        return this;
    }
    launched(crb_tensor_fill(elements, val, dims.size, nullptr), __FILE__, __LINE__);
    return this;
}

template <class Dist>
static Tensor *fill_random(Tensor *t, Dist dist, uint32 seed) {
    std::mt19937 gen(seed);
    if (t->deviceId == -1) {
        for (uint32 i = 0; i < t->dims.size; ++i) t->elements[i] = dist(gen);
        return t;
    }
    std::vector<float> tmp(t->dims.size);
    for (auto &v : tmp) v = dist(gen);
    if (hipMemcpy(t->elements, tmp.data(), sizeof(float) * tmp.size(), hipMemcpyHostToDevice) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    return t;
}

Tensor *Tensor::randNormal(float mean, float stddev, uint32 seed) {
    return fill_random(this, std::normal_distribution<float>(mean, stddev), seed);
}

Tensor *Tensor::randUniform(float min, float max, uint32 seed) {
    return fill_random(this, std::uniform_real_distribution<float>(min, max), seed);
}

float Tensor::get(uint32 offset) const {
    if (deviceId == -1) return elements[offset];
    float out = 0.0f;
    if (hipMemcpy(&out, elements + offset, sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    return out;
}

// ---- Parameter --------------------------------------------------------------------------------------
Parameter *Parameter::create(shape4 dims) {
    Parameter *p = new Parameter();
    p->A = Tensor::create(dims);
    p->dA = Tensor::create(dims);
    p->dAReserve = Tensor::create(dims);
    return p;
}

Parameter *Parameter::create(Tensor *src) {
    Parameter *p = new Parameter();
    p->A = src;
    p->dA = Tensor::create(src->dims);
    p->dAReserve = Tensor::create(src->dims);
    return p;
}

Parameter *Parameter::declare(shape4 dims) {
    Parameter *p = new Parameter();
    p->A = Tensor::declare(dims);
    p->dA = Tensor::declare(dims);
    p->dAReserve = Tensor::declare(dims);
    return p;
}

Parameter *Parameter::instantiate() {
    A->instantiate();
    dA->instantiate();
    dAReserve->instantiate();
    return this;
}

Parameter *Parameter::inherit(Parameter *src) {
    require(src->A->dims.size == A->dims.size, "Parameter::inherit: element counts differ");
    A->attach(src->A);
    dA->attach(src->dA);
    dAReserve->attach(src->dAReserve);
    return this;
}

void Parameter::eliminate() const {
    A->eliminate();
    dA->eliminate();
    dAReserve->eliminate();
}

}  // namespace seblas
