// Decoder table of the model file: per operand type id, one function that rebuilds the operand from its info record and
// one that creates its tensors and fills them from the parameter section (seio/modelcache/OperandCodecs.{cuh,cu}).
// Types this build has operands for: Linear, Conv2D (also read from the cuDNN convolution's id), BatchNorm, Softmax,
// ReLU, MaxPool2D and the two shortcut endpoints; get*Decoder returns nullptr for any other id.
#pragma once
#include <fstream>

#include "../../seann/operands/Conv2D.h"
#include "../../seann/operands/Elementwise.h"
#include "../../seann/operands/Linear.h"
#include "../../seann/operands/ShortcutEndpoint.h"

#define OPR_CUDNN_CONV2D 0xd002

namespace seio {
using namespace seann;

// `offset` is the running byte position in the info section (InfoDecoder) or the parameter section (ParamDecoder)
typedef OperandBase *(*InfoDecoder)(std::fstream *, uint64 &);
typedef void (*ParamDecoder)(std::fstream *, uint64 &, OperandBase *, OptimizerInfo *, shape4 inShape);

InfoDecoder getInfoDecoder(uint32 OPERAND_ID);
ParamDecoder getParamDecoder(uint32 OPERAND_ID);
}  // namespace seio
