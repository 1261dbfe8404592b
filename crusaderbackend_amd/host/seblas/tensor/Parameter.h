// seblas::Parameter — the (A, dA, dAReserve) same-shape triple of the reference
// (seblas/tensor/Parameter.cuh:11-77). inherit() aliases all three buffers onto another Parameter, which is
// how an operand's input X shares storage with the previous operand's output Y.
#pragma once
#include "Tensor.h"

namespace seblas {
class Parameter {
public:
    Tensor *A = nullptr;
    Tensor *dA = nullptr;
    Tensor *dAReserve = nullptr;

    static Parameter *create(shape4 dims);
    template <typename... Args>
    static Parameter *create(Args &&...args) { return create(shape4(std::forward<Args>(args)...)); }
    static Parameter *create(Tensor *src);
    static Parameter *declare(shape4 dims);
    template <typename... Args>
    static Parameter *declare(Args &&...args) { return declare(shape4(std::forward<Args>(args)...)); }

    Parameter *instantiate();
    Parameter *inherit(Parameter *src);  // requires equal element counts
    void eliminate() const;
};
}  // namespace seblas
