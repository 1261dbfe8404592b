// seio model files (".crseq"): saveSequence writes a Sequential's operand list, construction arguments and trainable
// tensors; loadSequence rebuilds the network from such a file (seio/modelcache/codec.cuh:18-74, codec.cu:8-97).
//
// Layout, all little-endian 4-byte words:
//   header      magic 0x7921aedf, operand count, epoch id
//   id table    one operand type id per top-level operand
//   info        per operand, its construction arguments (OperandBase::encodeInfo)
//   parameters  per operand, its trainable tensors as raw float32 (OperandBase::encodeNetParams)
// Optimizer state is not part of the file.
//
// Differences from the reference, none of which changes the bytes of a file:
//  * saveSequence replaces an existing file (the reference opens it in append mode, so a second save to the same name
//    leaves the first model at the front of the file, which is what loadSequence then reads);
//  * loadSequence accepts closing shortcut endpoints with branch operands: it moves past the branch's infos and creates
//    the branch's tensors for the shape that entered the opening endpoint. The reference's reader leaves the info cursor
//    inside the branch and indexes the branch list at -1 (OperandCodecs.cu:236-269), so it only reads networks whose
//    shortcuts are all identities;
//  * a file with a wrong magic number, an operand type this build has no operand for, or a truncated record throws
//    std::runtime_error instead of ending the process;
//  * type id 0xd002 (the reference's cuDNN convolution, same records as 0x0002) loads as a Conv2D.
#pragma once
#include <string>

#include "../../seann/containers/Sequential.h"
#include "OperandCodecs.h"

namespace seio {
using namespace seann;

struct FILE_HEAD {
    static constexpr uint32 MAGIC_NUMBER = 0x7921aedf;
    uint32 OPERAND_COUNT = 0;
    uint32 EPOCH_ID = 0;
    FILE_HEAD(uint32 operandCount, uint32 epochID) : OPERAND_COUNT(operandCount), EPOCH_ID(epochID) {}
    uint32 encode(std::fstream *fout) const;  // 12 bytes at the start of the stream
    void decode(std::fstream *fin);           // throws on a wrong magic number
};

void saveSequence(const char *fname, Sequential *seq, uint32 epochID);
Sequential *loadSequence(const char *fname, shape4 inShape, OptimizerInfo *info);
// The epoch id stored by saveSequence (loadSequence only logs it in the reference).
uint32 loadedEpochID(const char *fname);
// Text summary of a file's header and operand infos, one line per operand; touches no device memory.
std::string inspectSequence(const char *fname);
}  // namespace seio

// inspectSequence for callers without C++: writes at most cap - 1 characters and a terminator into out and returns the
// full length of the summary, or -1 (with the error text in out) if the file cannot be parsed.
extern "C" int seio_inspect_sequence(const char *fname, char *out, unsigned cap);
