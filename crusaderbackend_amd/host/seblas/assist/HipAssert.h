// Device-error convention of the seblas host layer: poll the HIP error state after an operation and throw
// std::runtime_error("line: <n> file: <f>") — the behaviour of assertCuda in the reference
// (seblas/assist/CudaAssert.cu:8-15). Shape errors throw std::invalid_argument (cuConv.cu:731-755).
#pragma once
#include <stdexcept>
#include <string>

namespace seblas {
void assertHip(const char *file, int line);
// Translates a C-ABI status (include/crusader_hip.h) into the reference's exception types; no-op on CRB_OK.
void throwOnStatus(int status, const char *file, int line);
}  // namespace seblas
