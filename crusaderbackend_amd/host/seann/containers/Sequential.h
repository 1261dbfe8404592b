// seann::Sequential — the linear container that owns the operand list, wires each operand's input to its predecessor's
// output and drives forward / backward / update (seann/containers/Sequential.{cuh,cu}). Dataset-driven `train` and logging are
// outside this build; seio::saveSequence / loadSequence write and read a network's model file.
#pragma once
#include <initializer_list>
#include <vector>

#include "../operands/OperandBase.h"

namespace seio {
struct Dataset;
}

namespace seann {

typedef void (*LossFunc)(Parameter *, Tensor *);
// Called by train() after every batch: epoch, batch id, training loss per sample, test loss per sample (0 when not tested).
typedef void (*TrainProgress)(uint32, uint32, float, float);
typedef float (*LossFuncCalc)(Parameter *, Tensor *, Tensor *);

class Sequential {
public:
    Parameter *netX;
    Parameter *netY{};
    LossFunc loss{};
    LossFuncCalc lossFW{};
    std::vector<OperandBase *> operands;
    uint32 OPERAND_COUNT;

    Sequential(shape4 inputShape, std::initializer_list<OperandBase *> list) : operands(list), OPERAND_COUNT(uint32(list.size())) {
        netX = Parameter::create(inputShape);
    }
    Sequential(shape4 inputShape, const std::vector<OperandBase *> &list) : operands(list), OPERAND_COUNT(uint32(list.size())) {
        netX = Parameter::create(inputShape);
    }

    void waive() const;                     // bind prev/next and inputs along the chain
    void construct(OptimizerInfo *info);    // create every operand's tensors, then bind
    void setLoss(LossFunc lossFunc, LossFuncCalc lossFWD) { loss = lossFunc, lossFW = lossFWD; }
    void randInit() const;
    Tensor *forward() const;
    Tensor *forward(Tensor *X) const;
    Tensor *inferenceForward() const;
    Tensor *inferenceForward(Tensor *X) const;
    Tensor *backward(Tensor *label) const;  // loss gradient, then xGrads + paramGrads from last to first
    void learn() const;
    void learnBatch() const;
    void zeroGrads() const;
    // The training loop (Sequential.cu:106-160): batches come from `data` (the next one is formed on another thread and
    // stream while this one trains), every mini-batch runs forward, backward, loss and learn; after each batch learnBatch,
    // and every TEST_FREQUENCY batches the test set's loss; when an epoch ends the gradients are cleared and, for epochs
    // 0, 5, 10, ..., the model is saved. The reference writes <cache dir>cache.log and cache.crseq at a hard-coded Windows
    // path and draws a console display; here the directory is an argument and progress goes to an optional callback.
    void train(seio::Dataset *data, bool WITH_TEST, uint32 TEST_FREQUENCY, const char *cacheDir = ".", TrainProgress progress = nullptr);

    // Optional shortcuts with no counterpart in the reference; results are unchanged.
    // pruneReserveFolds: after construct(), stop folding Y->dAReserve into Y->dA in the xGrads of operands into whose
    // reserve no operand of this network deposits anything (only shortcut endpoints do). An operand type of your own that
    // writes another operand's reserve must increment that operand's `reserveWriters` in its postWaiveInit.
    void pruneReserveFolds() const;
    // streamline: pruneReserveFolds plus letting every opening shortcut endpoint's output value alias its input (it only
    // passes it on), which removes one device copy per residual block from the forward pass, plus letting each convolution's
    // xGrads compute the filter gradient in the same launch as the input gradient (backward() calls the two as a pair) and
    // leave its last step, the sum of its partial results, to one launch for all convolutions at the end of backward(), plus
    // letting a batch normalisation or a closing shortcut endpoint compute the ReLU that follows it in its own passes.
    void streamline() const;
    // learnFused: the momentum step of every parameter in one kernel launch instead of one launch per parameter.
    void learnFused();

private:
    mutable std::vector<seblas::SliceSumItem> sliceItems;  // filter gradients left as partial sums by xGrads (streamline())
    void *fusedTable = nullptr;    // device copy of the parameter table used by learnFused
    std::vector<char> fusedHost;   // its host image, to detect changed rates
};
}  // namespace seann
