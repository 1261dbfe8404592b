#include "Dataset.h"

#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstring>
#include <stdexcept>

#include "../../../../include/crusader_hip.h"
#include "../../seblas/assist/HipAssert.h"

namespace seio {
namespace {
uint32 clockSeed() {
    return uint32(std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::system_clock::now().time_since_epoch()).count());
}
void hipOk(hipError_t e, const char *file, int line) {
    if (e != hipSuccess) assertHip(file, line);
}
#define HIP_OK(x) hipOk((x), __FILE__, __LINE__)
}  // namespace

// ---- Data ---------------------------------------------------------------------------------------------------------------
Data *Data::declare(shape4 dataShape, shape4 labelShape) {
    Data *out = new Data();
    out->X = Tensor::declare(dataShape);
    out->label = Tensor::declare(labelShape);
    return out;
}
Data *Data::instantiate() {
    X->instantiate(), label->instantiate();
    return this;
}
Data *Data::instantiateHost() {
    X->instantiateHost(), label->instantiateHost();
    return this;
}
Data *Data::inherit(Tensor *X0, Tensor *label0) {
    X->attach(X0), label->attach(label0);
    return this;
}

// ---- record readers -------------------------------------------------------------------------------------------------------
void Loader::loadData(Tensor *X, Tensor *label, const char *rootPath, const char *datasetName, uint32 offset) {
    if (X->deviceId != -1 || label->deviceId != -1) throw std::invalid_argument("Loader::loadData: host tensors expected");
    scratch.resize(X->dims.size);
    loadBytes(scratch.data(), label->elements, X->dims.size, label->dims.size, rootPath, datasetName, offset);
    for (uint32 i = 0; i < X->dims.size; i++) X->elements[i] = float(scratch[i]);
}

void CrdatLoader::loadBytes(uint8_t *pixels, float *label, uint32 dataSize, uint32 labelSize, const char *rootPath,
                            const char *datasetName, uint32 offset) {
    const std::string path = std::string(rootPath) + "/" + datasetName + ".crdat";
    if (path != openPath) {
        file.close();
        file.clear();
        file.open(path, std::ios::binary | std::ios::ate);
        if (!file) throw std::runtime_error("CrdatLoader: cannot open " + path);
        fileSize = uint64(file.tellg());
        openPath = path;
    }
    const uint64 operateSize = uint64(dataSize) + uint64(labelSize) * sizeof(float);
    if (uint64(offset) >= fileSize / operateSize) throw std::out_of_range("CrdatLoader: record past the end of " + path);
    file.seekg((long long)(uint64(offset) * operateSize), std::ios::beg);
    file.read(reinterpret_cast<char *>(pixels), dataSize);
    file.read(reinterpret_cast<char *>(label), std::streamsize(labelSize * sizeof(float)));
    if (!file) throw std::runtime_error("CrdatLoader: short read from " + path);
}

void CifarBinLoader::loadBytes(uint8_t *pixels, float *label, uint32 dataSize, uint32 labelSize, const char *, const char *,
                               uint32 offset) {
    const uint32 index = offset / recordsPerFile, within = offset % recordsPerFile;
    if (index >= files.size()) throw std::out_of_range("CifarBinLoader: record past the last file");
    if (int(index) != openIndex) {
        file.close();
        file.clear();
        file.open(files[index], std::ios::binary);
        if (!file) throw std::runtime_error("CifarBinLoader: cannot open " + files[index]);
        openIndex = int(index);
    }
    file.seekg((long long)(uint64(within) * (uint64(dataSize) + 1)), std::ios::beg);
    char cls = 0;
    file.read(&cls, 1);
    file.read(reinterpret_cast<char *>(pixels), dataSize);
    if (!file) {
        file.clear();
        throw std::out_of_range("CifarBinLoader: record past the end of " + files[index]);
    }
    if (uint32(uint8_t(cls)) >= labelSize) throw std::runtime_error("CifarBinLoader: class id exceeds the label size");
    for (uint32 i = 0; i < labelSize; i++) label[i] = 0.0f;
    label[uint8_t(cls)] = 1.0f;
}

// ---- fetcher ----------------------------------------------------------------------------------------------------------------
DataFetcher::DataFetcher(std::string rootPath, std::string datasetName, uint32 EPOCH_SIZE, uint32 TEST_SIZE, Loader *dataLoader,
                         uint32 seed)
    : ROOT_PATH(std::move(rootPath)), DATASET_NAME(std::move(datasetName)), EPOCH_SIZE(EPOCH_SIZE), TEST_SIZE(TEST_SIZE),
      dataLoader(dataLoader), remainedData(EPOCH_SIZE + TEST_SIZE), registry(EPOCH_SIZE + TEST_SIZE),
      generator(seed ? seed : clockSeed()) {
    if (!EPOCH_SIZE) throw std::invalid_argument("DataFetcher: empty epoch");
    for (uint32 i = 0; i < EPOCH_SIZE + TEST_SIZE; i++) registry[i] = i;
}

uint32 DataFetcher::draw(uint32 remaining) {
    std::uniform_int_distribution<uint32> distribution(0, remaining - 1);
    return distribution(generator);
}

uint32 DataFetcher::nextRecord() {
    const uint32 index = draw(remainedData);
    if (index >= remainedData) throw std::out_of_range("DataFetcher: drawn position outside the remaining records");
    const uint32 selected = registry[index];
    std::memmove(&registry[index], &registry[index + 1], sizeof(uint32) * (remainedData - 1 - index));
    registry[remainedData - 1] = selected;
    remainedData--;
    if (remainedData == 0) remainedData = EPOCH_SIZE;
    return selected;
}

void DataFetcher::fetchTrain(Data **dataset, uint32 step) {
    for (uint32 i = 0; i < step; i++)
        dataLoader->loadData(dataset[i]->X, dataset[i]->label, ROOT_PATH.c_str(), DATASET_NAME.c_str(), nextRecord());
}

void DataFetcher::fetchTrainBytes(uint8_t *pixels, float *labels, uint32 dataSize, uint32 labelSize, uint32 step) {
    for (uint32 i = 0; i < step; i++)
        dataLoader->loadBytes(pixels + size_t(i) * dataSize, labels + size_t(i) * labelSize, dataSize, labelSize, ROOT_PATH.c_str(),
                              DATASET_NAME.c_str(), nextRecord());
}

void DataFetcher::fetchTest(Tensor *data, Tensor *label) {  // DataFetcher.cu:49-70: a draw that consumes nothing
    dataLoader->loadData(data, label, ROOT_PATH.c_str(), DATASET_NAME.c_str(), registry[draw(remainedData)]);
}

// ---- transforms, augmentations ------------------------------------------------------------------------------------------------
int DistribNorm::kind() const { return CRB_NORM_DISTRIBUTION; }
int UniformNorm::kind() const { return CRB_NORM_UNIFORM; }

void RandFlipW::decide(ImageAug &aug, std::default_random_engine &generator) {
    std::uniform_int_distribution<uint32> flipProp(0, 1);
    if (flipProp(generator)) aug.flags |= CRB_AUG_MIRROR;
}

void RandCorp::decide(ImageAug &aug, std::default_random_engine &generator) {
    std::uniform_int_distribution<uint32> hDist(0, 2 * padH), wDist(0, 2 * padW);
    aug.dh = int(hDist(generator)) - int(padH);
    aug.dw = int(wDist(generator)) - int(padW);
    aug.flags |= CRB_AUG_SHIFT;
}

// ---- Dataset ----------------------------------------------------------------------------------------------------------------
Dataset *Dataset::construct(uint32 batchSize, uint32 miniBatchSize, uint32 epochSize, uint32 maxEpoch, shape4 dataShape,
                            shape4 labelShape, uint32 seed) {
    if (!batchSize || !epochSize || batchSize > epochSize || !miniBatchSize || batchSize % miniBatchSize)
        throw std::invalid_argument("Dataset::construct: batch, mini-batch and epoch sizes do not fit");  // Dataset.cu:22-34
    if (dataShape.n != 1 || labelShape.n != 1) throw std::invalid_argument("Dataset::construct: per-sample shapes expected");
    Dataset *out = new Dataset();
    out->BATCH_SIZE = batchSize, out->EPOCH_SIZE = epochSize, out->MAX_EPOCH = maxEpoch, out->MINI_BATCH_SIZE = miniBatchSize;
    out->dataShape = dataShape, out->labelShape = labelShape;
    out->generator.seed(seed ? seed : clockSeed());
    const size_t xBytes = size_t(batchSize) * dataShape.size, labFloats = size_t(batchSize) * labelShape.size;
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&out->pinnedPixels), xBytes, hipHostMallocDefault));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&out->pinnedLabels), labFloats * sizeof(float), hipHostMallocDefault));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&out->pinnedAug), sizeof(ImageAug) * batchSize, hipHostMallocDefault));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&out->devPixels), xBytes));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&out->devAug), sizeof(ImageAug) * batchSize));
    hipStream_t s;
    HIP_OK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    out->stream = s;
    const uint32 minis = batchSize / miniBatchSize;
    const shape4 procData(miniBatchSize, dataShape.c, dataShape.h, dataShape.w), procLabel(miniBatchSize, labelShape.c, labelShape.h, labelShape.w);
    for (int side = 0; side < 2; side++) {
        HIP_OK(hipMalloc(reinterpret_cast<void **>(&out->devX[side]), xBytes * sizeof(float)));
        HIP_OK(hipMalloc(reinterpret_cast<void **>(&out->devLabel[side]), labFloats * sizeof(float)));
        out->dataBatch[side] = new Data *[minis];
        for (uint32 i = 0; i < minis; i++) {
            Data *d = Data::declare(procData, procLabel);
            d->X->attach(out->devX[side] + size_t(i) * procData.size, 0);
            d->label->attach(out->devLabel[side] + size_t(i) * procLabel.size, 0);
            out->dataBatch[side][i] = d;
        }
    }
    return out;
}

void Dataset::setProcSteps(std::initializer_list<DataTransformer *> steps) {
    if (steps.size() > 1) throw std::invalid_argument("Dataset::setProcSteps: at most one transform");
    preProc = steps.size() ? *steps.begin() : nullptr;
}

void Dataset::setAugmentSteps(std::initializer_list<DataAugmentor *> steps) { augmentations.assign(steps.begin(), steps.end()); }

void Dataset::genBatch() {  // Dataset.cu:63-85
    if (!fetcher) throw std::invalid_argument("Dataset::genBatch: no data fetcher");
    const int side = int(batchID % 2);
    hipStream_t s = hipStream_t(stream);
    fetcher->fetchTrainBytes(pinnedPixels, pinnedLabels, dataShape.size, labelShape.size, BATCH_SIZE);
    augHost.assign(BATCH_SIZE, ImageAug());
    // the reference decides mini-batch by mini-batch, each augmentation over the whole mini-batch before the next one
    for (uint32 mb = 0; mb < BATCH_SIZE / MINI_BATCH_SIZE; mb++)
        for (DataAugmentor *step : augmentations)
            for (uint32 i = 0; i < MINI_BATCH_SIZE; i++) step->decide(augHost[size_t(mb) * MINI_BATCH_SIZE + i], generator);
    const bool anyAug = !augmentations.empty();
    if (anyAug) {
        std::memcpy(pinnedAug, augHost.data(), sizeof(ImageAug) * BATCH_SIZE);
        HIP_OK(hipMemcpyAsync(devAug, pinnedAug, sizeof(ImageAug) * BATCH_SIZE, hipMemcpyHostToDevice, s));
    }
    HIP_OK(hipMemcpyAsync(devPixels, pinnedPixels, size_t(BATCH_SIZE) * dataShape.size, hipMemcpyHostToDevice, s));
    HIP_OK(hipMemcpyAsync(devLabel[side], pinnedLabels, size_t(BATCH_SIZE) * labelShape.size * sizeof(float), hipMemcpyHostToDevice, s));
    static_assert(sizeof(ImageAug) == sizeof(crb_image_aug), "augmentation record layout");
    throwOnStatus(crb_images_from_bytes(devPixels, devX[side], BATCH_SIZE, dataShape.c, dataShape.h, dataShape.w,
                                        preProc ? preProc->kind() : CRB_NORM_NONE, preProc ? preProc->p0() : 0.0f,
                                        preProc ? preProc->p1() : 0.0f, anyAug ? reinterpret_cast<const crb_image_aug *>(devAug) : nullptr, s),
                  __FILE__, __LINE__);
    HIP_OK(hipStreamSynchronize(s));  // the batch is complete, and the pinned buffers free again, when genBatch returns
    batchID++;
    epochID = uint32((uint64(batchID) * BATCH_SIZE) / EPOCH_SIZE);
}

void Dataset::allocTestSet() {
    if (!fetcher) throw std::invalid_argument("Dataset::allocTestSet: no data fetcher");
    const uint32 n = fetcher->TEST_SIZE;
    if (!n || n % MINI_BATCH_SIZE) throw std::invalid_argument("Dataset::allocTestSet: test size must be a positive multiple of the mini-batch size");
    TEST_SIZE = n;
    const size_t xBytes = size_t(n) * dataShape.size, labFloats = size_t(n) * labelShape.size;
    uint8_t *hostPix = nullptr, *devPix = nullptr;
    float *hostLab = nullptr, *devXt = nullptr, *devLt = nullptr;
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&hostPix), xBytes, hipHostMallocDefault));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&hostLab), labFloats * sizeof(float), hipHostMallocDefault));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&devPix), xBytes));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&devXt), xBytes * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&devLt), labFloats * sizeof(float)));
    Tensor *one = Tensor::createHost(dataShape), *lab = Tensor::createHost(labelShape);
    std::vector<uint8_t> bytes(dataShape.size);
    for (uint32 i = 0; i < n; i++) {  // fetchTest hands out floats of byte values: exact to turn back
        fetcher->fetchTest(one, lab);
        for (uint32 k = 0; k < dataShape.size; k++) hostPix[size_t(i) * dataShape.size + k] = uint8_t(one->elements[k]);
        std::memcpy(hostLab + size_t(i) * labelShape.size, lab->elements, sizeof(float) * labelShape.size);
    }
    one->eliminateHost(), lab->eliminateHost();
    hipStream_t s = hipStream_t(stream);
    HIP_OK(hipMemcpyAsync(devPix, hostPix, xBytes, hipMemcpyHostToDevice, s));
    HIP_OK(hipMemcpyAsync(devLt, hostLab, labFloats * sizeof(float), hipMemcpyHostToDevice, s));
    throwOnStatus(crb_images_from_bytes(devPix, devXt, n, dataShape.c, dataShape.h, dataShape.w, preProc ? preProc->kind() : CRB_NORM_NONE,
                                        preProc ? preProc->p0() : 0.0f, preProc ? preProc->p1() : 0.0f, nullptr, s),
                  __FILE__, __LINE__);
    HIP_OK(hipStreamSynchronize(s));
    HIP_OK(hipHostFree(hostPix));
    HIP_OK(hipHostFree(hostLab));
    HIP_OK(hipFree(devPix));
    const uint32 minis = n / MINI_BATCH_SIZE;
    const shape4 procData(MINI_BATCH_SIZE, dataShape.c, dataShape.h, dataShape.w), procLabel(MINI_BATCH_SIZE, labelShape.c, labelShape.h, labelShape.w);
    testset = new Data *[minis];
    for (uint32 i = 0; i < minis; i++) {
        Data *d = Data::declare(procData, procLabel);
        d->X->attach(devXt + size_t(i) * procData.size, 0);
        d->label->attach(devLt + size_t(i) * procLabel.size, 0);
        testset[i] = d;
    }
}

std::thread Dataset::genBatchAsync() {
    return std::thread([this] { genBatch(); });
}
}  // namespace seio
