// Model-file writer and reader; the per-operand records live with their decoders in this file.
#include "codec.h"

#include <hip/hip_runtime_api.h>

#include <cstring>
#include <map>
#include <sstream>
#include <stdexcept>
#include <vector>

#include "../../seblas/assist/HipAssert.h"

namespace {
using seblas::uint32;
using seblas::uint64;

void put(std::fstream *f, uint32 v) { f->write(reinterpret_cast<const char *>(&v), sizeof(uint32)); }

uint32 get(std::fstream *f) {
    uint32 v = 0;
    f->read(reinterpret_cast<char *>(&v), sizeof(uint32));
    if (!*f) throw std::runtime_error("crseq: file ends inside a record");
    return v;
}


// shape that entered each opening shortcut endpoint while a file's parameter section is read, by uuid
thread_local std::map<uint32, seblas::shape4> openShapes;
}  // namespace

// ---- NetParam records (NetParam.cuh:45-102) ---------------------------------------------------------------------------
namespace seann {
uint32 NetParam::encodeNetParamInfo(std::fstream *fout, uint64 offset) const {
    fout->seekp((long long)offset);
    const shape4 &d = A->A->dims;
    put(fout, d.n), put(fout, d.c), put(fout, d.h), put(fout, d.w);
    return 16;
}

uint32 NetParam::encodeNetParamData(std::fstream *fout, uint64 offset) const {
    const size_t count = A->A->dims.size;
    std::vector<float> host(count);
    if (hipMemcpy(host.data(), A->A->elements, count * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    fout->seekp((long long)offset);
    fout->write(reinterpret_cast<const char *>(host.data()), (long long)(count * sizeof(float)));
    return uint32(count * sizeof(float));
}

NetParam *NetParam::decodeNetParamInfo(std::fstream *fin, uint64 &offset, OptimizerInfo *info) {
    fin->seekg((long long)offset);
    uint32 n = get(fin), c = get(fin), h = get(fin), w = get(fin);
    offset += 16;
    return new NetParam(info, n, c, h, w);
}

NetParam *NetParam::decodeNetParamData(std::fstream *fin, uint64 &offset, NetParam *param) {
    const size_t count = param->A->A->dims.size;
    std::vector<float> host(count);
    fin->seekg((long long)offset);
    fin->read(reinterpret_cast<char *>(host.data()), (long long)(count * sizeof(float)));
    if (!*fin) throw std::runtime_error("crseq: file ends inside a parameter tensor");
    if (hipMemcpy(param->A->A->elements, host.data(), count * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
        assertHip(__FILE__, __LINE__);
    offset += count * sizeof(float);
    return param;
}

// ---- operand records --------------------------------------------------------------------------------------------------
uint32 Conv2D::encodeInfo(std::fstream *fout, uint64 offset) {  // Conv2D.cu:59-71
    uint64 running = offset;
    if (filter) {
        running += filter->encodeNetParamInfo(fout, running);
    } else {  // not constructed yet: the filter shape the operand was declared with
        fout->seekp((long long)running);
        put(fout, filterShape.n), put(fout, filterShape.c), put(fout, filterShape.h), put(fout, filterShape.w);
        running += 16;
    }
    fout->seekp((long long)running);
    put(fout, strideH), put(fout, strideW), put(fout, padH), put(fout, padW), put(fout, WITH_BIAS ? 1u : 0u);
    running += sizeof(uint32) * 5;
    return uint32(running - offset);
}

uint32 Conv2D::encodeNetParams(std::fstream *fout, uint64 offset) {  // Conv2D.cu:73-80
    uint64 running = offset;
    running += filter->encodeNetParamData(fout, running);
    if (WITH_BIAS) running += bias->encodeNetParamData(fout, running);
    return uint32(running - offset);
}

uint32 Linear::encodeInfo(std::fstream *fout, uint64 offset) {  // Linear.cu:62-68
    fout->seekp((long long)offset);
    put(fout, OUTPUT_SIZE);
    return sizeof(uint32);
}

uint32 Linear::encodeNetParams(std::fstream *fout, uint64 offset) {  // Linear.cu:70-75
    uint64 running = offset;
    running += weights->encodeNetParamData(fout, running);
    running += biases->encodeNetParamData(fout, running);
    return uint32(running - offset);
}

uint32 MaxPool2D::encodeInfo(std::fstream *fout, uint64 offset) {  // MaxPool2D.cu:22-29
    fout->seekp((long long)offset);
    put(fout, strideH), put(fout, strideW), put(fout, rangeH), put(fout, rangeW);
    return sizeof(uint32) * 4;
}

uint32 BatchNorm::encodeNetParams(std::fstream *fout, uint64 offset) {  // BatchNorm.cu:50-55
    uint64 running = offset;
    running += beta->encodeNetParamData(fout, running);
    running += gamma->encodeNetParamData(fout, running);
    return uint32(running - offset);
}

uint32 ShortcutEndpoint::encodeInfo(std::fstream *fout, uint64 offset) {  // ShortcutEndpoint.cu:151-167
    uint64 running = offset;
    fout->seekp((long long)running);
    put(fout, uuid), put(fout, operandCount);
    running += sizeof(uint32) * 2;
    if (isContainer) {
        for (OperandBase *op : branchOperands) put(fout, op->OPERAND_ID()), running += sizeof(uint32);
        for (OperandBase *op : branchOperands) running += op->encodeInfo(fout, running);
    }
    return uint32(running - offset);
}

uint32 ShortcutEndpoint::encodeNetParams(std::fstream *fout, uint64 offset) {  // ShortcutEndpoint.cu:169-177
    uint64 running = offset;
    for (OperandBase *op : branchOperands) running += op->encodeNetParams(fout, running);
    return uint32(running - offset);
}

// bytes encodeInfo writes: uuid, count, the branch's id table and infos
uint32 ShortcutEndpoint::getInfoEncodingSize() {
    uint32 size = sizeof(uint32) * 2;
    for (OperandBase *op : branchOperands) size += uint32(sizeof(uint32)) + op->getInfoEncodingSize();
    return size;
}

uint32 ShortcutEndpoint::getNetParamsEncodingSize() {
    uint32 size = 0;
    for (OperandBase *op : branchOperands) size += op->getNetParamsEncodingSize();
    return size;
}
}  // namespace seann

// ---- decoders (OperandCodecs.cu) ----------------------------------------------------------------------------------------
namespace seio {
namespace {
void initOnly(std::fstream *, uint64 &, OperandBase *opr, OptimizerInfo *info, shape4 inShape) { opr->initNetParams(info, inShape); }

OperandBase *decSoftmaxInfo(std::fstream *, uint64 &) { return new Softmax(); }
OperandBase *decReluInfo(std::fstream *, uint64 &) { return new ReLU(); }
OperandBase *decBatchNormInfo(std::fstream *, uint64 &) { return new BatchNorm(); }

OperandBase *decLinearInfo(std::fstream *fin, uint64 &offset) {  // :17-24
    fin->seekg((long long)offset);
    uint32 out = get(fin);
    offset += sizeof(uint32);
    return new Linear(out);
}

void decLinearParam(std::fstream *fin, uint64 &offset, OperandBase *opr, OptimizerInfo *info, shape4 inShape) {  // :26-31
    auto *linear = static_cast<Linear *>(opr);
    linear->initNetParams(info, inShape);
    NetParam::decodeNetParamData(fin, offset, linear->weights);
    NetParam::decodeNetParamData(fin, offset, linear->biases);
}

OperandBase *decConv2DInfo(std::fstream *fin, uint64 &offset) {  // :45-64, :175-195
    fin->seekg((long long)offset);
    uint32 fn = get(fin), fc = get(fin), fh = get(fin), fw = get(fin);
    uint32 strideH = get(fin), strideW = get(fin), padH = get(fin), padW = get(fin), n = get(fin);
    offset += sizeof(uint32) * 9;
    return new Conv2D(shape4(fn, fc, fh, fw), strideH, strideW, padH, padW, n > 0);
}

void decConv2DParam(std::fstream *fin, uint64 &offset, OperandBase *opr, OptimizerInfo *info, shape4 inShape) {  // :66-75
    auto *conv = static_cast<Conv2D *>(opr);
    conv->initNetParams(info, inShape);
    NetParam::decodeNetParamData(fin, offset, conv->filter);
    if (conv->WITH_BIAS) NetParam::decodeNetParamData(fin, offset, conv->bias);
}

void decBatchNormParam(std::fstream *fin, uint64 &offset, OperandBase *opr, OptimizerInfo *info, shape4 inShape) {  // :81-86
    auto *bn = static_cast<BatchNorm *>(opr);
    bn->initNetParams(info, inShape);
    NetParam::decodeNetParamData(fin, offset, bn->beta);
    NetParam::decodeNetParamData(fin, offset, bn->gamma);
}

OperandBase *decMaxPool2DInfo(std::fstream *fin, uint64 &offset) {  // :88-97
    fin->seekg((long long)offset);
    uint32 strideH = get(fin), strideW = get(fin), rangeH = get(fin), rangeW = get(fin);
    offset += sizeof(uint32) * 4;
    return new MaxPool2D(strideH, strideW, rangeH, rangeW);
}

OperandBase *decShortcutBegInfo(std::fstream *fin, uint64 &offset) {  // :220-229
    fin->seekg((long long)offset);
    uint32 uuid = get(fin);
    get(fin);  // branch operand count: always 0 for an opening endpoint
    offset += sizeof(uint32) * 2;
    return new ShortcutEndpoint(false, uuid, {});
}

void decShortcutBegParam(std::fstream *, uint64 &, OperandBase *opr, OptimizerInfo *info, shape4 inShape) {
    opr->initNetParams(info, inShape);
    openShapes[static_cast<ShortcutEndpoint *>(opr)->uuid] = inShape;
}

OperandBase *decShortcutEndInfo(std::fstream *fin, uint64 &offset) {  // :236-259
    fin->seekg((long long)offset);
    uint32 uuid = get(fin), count = get(fin);
    offset += sizeof(uint32) * 2;
    std::vector<OperandBase *> branch;
    uint64 subInfoOffset = offset + sizeof(uint32) * count;
    for (uint32 i = 0; i < count; i++) {
        fin->seekg((long long)offset);
        uint32 id = get(fin);
        offset += sizeof(uint32);
        InfoDecoder dec = getInfoDecoder(id);
        if (!dec) throw std::runtime_error("crseq: no operand for type id " + std::to_string(id) + " in a shortcut branch");
        branch.push_back(dec(fin, subInfoOffset));
    }
    offset = subInfoOffset;  // past the branch's infos: the next operand's info starts here
    return new ShortcutEndpoint(true, uuid, branch);
}

void decShortcutEndParam(std::fstream *fin, uint64 &offset, OperandBase *opr, OptimizerInfo *info, shape4 inShape) {  // :261-269
    auto *shortcut = static_cast<ShortcutEndpoint *>(opr);
    if (shortcut->operandCount > 0) {
        auto it = openShapes.find(shortcut->uuid);
        if (it == openShapes.end()) throw std::runtime_error("crseq: closing shortcut endpoint without an opening one");
        shape4 s = it->second;
        for (OperandBase *op : shortcut->branchOperands) {
            getParamDecoder(op->OPERAND_ID())(fin, offset, op, info, s);
            s = op->Y->A->dims;
        }
        shortcut->branchInitialised = true;
    }
    shortcut->initNetParams(info, inShape);
}
}  // namespace

InfoDecoder getInfoDecoder(uint32 OPERAND_ID) {
    switch (OPERAND_ID) {
        case OPR_SEBLAS_SOFTMAX: return decSoftmaxInfo;
        case OPR_SEBLAS_CONV2D: return decConv2DInfo;
        case OPR_CUDNN_CONV2D: return decConv2DInfo;
        case OPR_SEBLAS_LINEAR: return decLinearInfo;
        case OPR_SEBLAS_RELU: return decReluInfo;
        case OPR_SEBLAS_MAXPOOL2D: return decMaxPool2DInfo;
        case OPR_SEBLAS_BATCHNORM: return decBatchNormInfo;
        case OPR_CTRL_SHORTCUTENDPOINT_BEG: return decShortcutBegInfo;
        case OPR_CTRL_SHORTCUTENDPOINT_END: return decShortcutEndInfo;
        default: return nullptr;
    }
}

ParamDecoder getParamDecoder(uint32 OPERAND_ID) {
    switch (OPERAND_ID) {
        case OPR_SEBLAS_SOFTMAX: return initOnly;
        case OPR_SEBLAS_CONV2D: return decConv2DParam;
        case OPR_CUDNN_CONV2D: return decConv2DParam;
        case OPR_SEBLAS_LINEAR: return decLinearParam;
        case OPR_SEBLAS_RELU: return initOnly;
        case OPR_SEBLAS_MAXPOOL2D: return initOnly;
        case OPR_SEBLAS_BATCHNORM: return decBatchNormParam;
        case OPR_CTRL_SHORTCUTENDPOINT_BEG: return decShortcutBegParam;
        case OPR_CTRL_SHORTCUTENDPOINT_END: return decShortcutEndParam;
        default: return nullptr;
    }
}

// ---- file level (codec.cuh:40-74, codec.cu:8-97) ------------------------------------------------------------------------
uint32 FILE_HEAD::encode(std::fstream *fout) const {
    fout->seekp(0);
    put(fout, MAGIC_NUMBER), put(fout, OPERAND_COUNT), put(fout, EPOCH_ID);
    return sizeof(uint32) * 3;
}

void FILE_HEAD::decode(std::fstream *fin) {
    fin->seekg(0);
    if (get(fin) != MAGIC_NUMBER) throw std::runtime_error("crseq: wrong magic number (not a model file)");
    OPERAND_COUNT = get(fin);
    EPOCH_ID = get(fin);
}

void saveSequence(const char *fname, Sequential *seq, uint32 epochID) {
    std::fstream fout(fname, std::ios::binary | std::ios::out | std::ios::trunc);
    if (!fout) throw std::runtime_error(std::string("crseq: cannot open for writing: ") + fname);
    FILE_HEAD header(seq->OPERAND_COUNT, epochID);
    uint64 offset = header.encode(&fout);
    fout.seekp((long long)offset);
    for (uint32 i = 0; i < seq->OPERAND_COUNT; i++) {
        put(&fout, seq->operands[i]->OPERAND_ID());
        offset += sizeof(uint32);
    }
    for (uint32 i = 0; i < seq->OPERAND_COUNT; i++) offset += seq->operands[i]->encodeInfo(&fout, offset);
    for (uint32 i = 0; i < seq->OPERAND_COUNT; i++) offset += seq->operands[i]->encodeNetParams(&fout, offset);
    fout.flush();
    if (!fout) throw std::runtime_error(std::string("crseq: write failed: ") + fname);
}

namespace {
// header and info section -> operands without tensors; returns the byte offset of the parameter section
uint64 readOperands(std::fstream *fin, FILE_HEAD &header, std::vector<OperandBase *> &operands) {
    header.decode(fin);
    uint64 offset = 12;
    uint64 operandInfoOffset = offset + sizeof(uint32) * uint64(header.OPERAND_COUNT);
    for (uint32 i = 0; i < header.OPERAND_COUNT; i++) {
        fin->seekg((long long)offset);
        uint32 id = get(fin);
        offset += sizeof(uint32);
        InfoDecoder dec = getInfoDecoder(id);
        if (!dec) {
            std::ostringstream msg;
            msg << "crseq: no operand for type id 0x" << std::hex << id;
            throw std::runtime_error(msg.str());
        }
        operands.push_back(dec(fin, operandInfoOffset));
    }
    return operandInfoOffset;
}
}  // namespace

Sequential *loadSequence(const char *fname, shape4 inShape, OptimizerInfo *info) {
    std::fstream fin(fname, std::ios::binary | std::ios::in);
    if (!fin) throw std::runtime_error(std::string("crseq: cannot open: ") + fname);
    FILE_HEAD header(0, 0);
    std::vector<OperandBase *> operands;
    uint64 offset = readOperands(&fin, header, operands);
    if (operands.empty()) throw std::runtime_error("crseq: the file holds no operands");

    openShapes.clear();
    for (uint32 i = 0; i < header.OPERAND_COUNT; i++) {
        getParamDecoder(operands[i]->OPERAND_ID())(&fin, offset, operands[i], info, i > 0 ? operands[i - 1]->Y->A->dims : inShape);
        operands[i]->operandID = i;
    }
    openShapes.clear();

    auto *seq = new Sequential(inShape, operands);
    operands[0]->X->inherit(seq->netX);
    seq->netY = Parameter::declare(operands[seq->OPERAND_COUNT - 1]->Y->A->dims)->inherit(operands[seq->OPERAND_COUNT - 1]->Y);
    seq->waive();
    for (uint32 i = 0; i < seq->OPERAND_COUNT; i++) operands[i]->postWaiveInit(info);
    return seq;
}

uint32 loadedEpochID(const char *fname) {
    std::fstream fin(fname, std::ios::binary | std::ios::in);
    if (!fin) throw std::runtime_error(std::string("crseq: cannot open: ") + fname);
    FILE_HEAD header(0, 0);
    header.decode(&fin);
    return header.EPOCH_ID;
}

namespace {
void describe(std::ostringstream &out, OperandBase *op, int depth) {
    out << std::string(size_t(depth) * 2, ' ');
    if (auto *c = dynamic_cast<Conv2D *>(op)) {
        out << "conv2d filter=" << c->filterShape.n << "," << c->filterShape.c << "," << c->filterShape.h << "," << c->filterShape.w
            << " stride=" << c->strideH << "," << c->strideW << " pad=" << c->padH << "," << c->padW << " bias=" << (c->WITH_BIAS ? 1 : 0) << "\n";
    } else if (auto *l = dynamic_cast<Linear *>(op)) {
        out << "linear out=" << l->OUTPUT_SIZE << "\n";
    } else if (auto *p = dynamic_cast<MaxPool2D *>(op)) {
        out << "maxpool2d stride=" << p->strideH << "," << p->strideW << " range=" << p->rangeH << "," << p->rangeW << "\n";
    } else if (dynamic_cast<BatchNorm *>(op)) {
        out << "batchnorm\n";
    } else if (dynamic_cast<ReLU *>(op)) {
        out << "relu\n";
    } else if (dynamic_cast<Softmax *>(op)) {
        out << "softmax\n";
    } else if (auto *s = dynamic_cast<ShortcutEndpoint *>(op)) {
        out << (s->isContainer ? "shortcut_end" : "shortcut_beg") << " uuid=" << s->uuid << " branch=" << s->operandCount << "\n";
        for (OperandBase *b : s->branchOperands) describe(out, b, depth + 1);
    }
}
}  // namespace

std::string inspectSequence(const char *fname) {
    std::fstream fin(fname, std::ios::binary | std::ios::in);
    if (!fin) throw std::runtime_error(std::string("crseq: cannot open: ") + fname);
    FILE_HEAD header(0, 0);
    std::vector<OperandBase *> operands;
    uint64 paramOffset = readOperands(&fin, header, operands);
    fin.seekg(0, std::ios::end);
    std::ostringstream out;
    out << "operands=" << header.OPERAND_COUNT << " epoch=" << header.EPOCH_ID << " params_at=" << paramOffset
        << " param_bytes=" << (uint64(fin.tellg()) - paramOffset) << "\n";
    for (OperandBase *op : operands) describe(out, op, 0);
    for (OperandBase *op : operands) {
        if (auto *s = dynamic_cast<ShortcutEndpoint *>(op))
            for (OperandBase *b : s->branchOperands) delete b;
        delete op;
    }
    return out.str();
}
}  // namespace seio

extern "C" int seio_inspect_sequence(const char *fname, char *out, unsigned cap) {
    std::string text;
    int rc = 0;
    try {
        text = seio::inspectSequence(fname);
        rc = int(text.size());
    } catch (const std::exception &e) {
        text = e.what();
        rc = -1;
    }
    if (out && cap) {
        size_t n = text.size() < size_t(cap) - 1 ? text.size() : size_t(cap) - 1;
        std::memcpy(out, text.data(), n);
        out[n] = 0;
    }
    return rc;
}
