// seio data pipeline from a dataset file to mini-batches in device memory: record readers, the fetcher that samples
// records without replacement, the per-image normalising transform and the mirror / shift augmentations, and the
// Dataset that forms batches (seio/data/DataLoader.{cuh,cu}, DataFetcher.{cuh,cu}, DataTransform.{cuh,cu},
// DataAugmentor.{cuh,cu}, Dataset.{cuh,cu}).
//
// The reference converts, normalises and augments every image in host loops and uploads floats. Here the records'
// pixel bytes go to pinned host memory as they are, the whole batch is uploaded as bytes (a quarter of the volume), and
// one kernel launch (crb_images_from_bytes) converts, normalises, mirrors and shifts all of it into the device buffer
// the mini-batches are views of. The arithmetic per value is the reference's; so are the record layouts and the
// sampling rule. Differences: directory separators are '/', the random generators can be seeded (seed 0 = from the
// clock, as the reference always does), the mirror is a true mirror (the reference stores to column W - w, one past
// the row, DataAugmentor.cu:78-80), transforms and augmentations are descriptions consumed by the kernel rather than host
// functions, at most one transform per dataset, and the image loader for directories of pictures (OpenCV) is not built.
#pragma once
#include <cstdint>
#include <fstream>
#include <initializer_list>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../seblas/tensor/Tensor.h"

namespace seio {
using namespace seblas;

// One sample or one mini-batch: values and labels (seio/data/Data.cuh:13-45).
struct Data {
    Tensor *X = nullptr;
    Tensor *label = nullptr;
    static Data *declare(shape4 dataShape, shape4 labelShape);
    Data *instantiate();      // device
    Data *instantiateHost();  // pinned host
    Data *inherit(Tensor *X0, Tensor *label0);
};

// Reads one record: `pixels` receives the stored bytes (dataSize of them), `label` the label values (labelSize floats).
struct Loader {
    virtual ~Loader() = default;
    virtual void loadBytes(uint8_t *pixels, float *label, uint32 dataSize, uint32 labelSize, const char *rootPath,
                           const char *datasetName, uint32 offset) = 0;
    // The reference's form: a host tensor of floats, X[i] = (float) byte i (DataLoader.cu:34-36).
    void loadData(Tensor *X, Tensor *label, const char *rootPath, const char *datasetName, uint32 offset);

private:
    std::vector<uint8_t> scratch;
};

// <root>/<name>.crdat: records of dataSize pixel bytes followed by labelSize float32 label values, no header
// (CrdatLoader::loadData, DataLoader.cu:14-41). Throws std::out_of_range for a record past the end of the file.
struct CrdatLoader : public Loader {
    void loadBytes(uint8_t *pixels, float *label, uint32 dataSize, uint32 labelSize, const char *rootPath, const char *datasetName,
                   uint32 offset) override;

private:
    std::ifstream file;
    std::string openPath;
    uint64 fileSize = 0;
};

// CIFAR-10 binary batches: records of 1 label byte followed by 3072 pixel bytes (three 32 x 32 planes). Record ids run
// through the files in the order given: <root>/<name>1.bin ... <name>5.bin style lists are passed as full file names.
// The label becomes a one-hot vector of labelSize values. This is what the archived training programs load with
// fetchCIFAR(dataset, path, fileIndex) (archive/Resnet56:276-282).
struct CifarBinLoader : public Loader {
    explicit CifarBinLoader(std::vector<std::string> files, uint32 recordsPerFile = 10000)
        : files(std::move(files)), recordsPerFile(recordsPerFile) {}
    void loadBytes(uint8_t *pixels, float *label, uint32 dataSize, uint32 labelSize, const char *rootPath, const char *datasetName,
                   uint32 offset) override;

private:
    std::vector<std::string> files;
    uint32 recordsPerFile;
    std::ifstream file;
    int openIndex = -1;
};

// Samples record ids without replacement (DataFetcher.cuh:24-49, DataFetcher.cu:10-47): the registry holds ids
// 0 .. EPOCH_SIZE + TEST_SIZE - 1, all of them remaining at first; a fetch draws a position among the remaining ones,
// takes that id and moves it behind the remaining part; when nothing remains, EPOCH_SIZE ids remain again.
class DataFetcher {
public:
    std::string ROOT_PATH, DATASET_NAME;
    uint32 EPOCH_SIZE, TEST_SIZE;
    Loader *dataLoader;
    uint32 remainedData;
    std::vector<uint32> registry;

    DataFetcher(std::string rootPath, std::string datasetName, uint32 EPOCH_SIZE, uint32 TEST_SIZE, Loader *dataLoader,
                uint32 seed = 0);
    virtual ~DataFetcher() = default;
    virtual uint32 draw(uint32 remaining);  // a position in [0, remaining); override to supply a fixed sequence
    uint32 nextRecord();                    // one sampling step: the record id to load
    void fetchTrain(Data **dataset, uint32 step);  // the reference's form: host Data of floats
    void fetchTrainBytes(uint8_t *pixels, float *labels, uint32 dataSize, uint32 labelSize, uint32 step);
    void fetchTest(Tensor *data, Tensor *label);

private:
    std::default_random_engine generator;
};

// Per-image normalisation applied when a batch is formed (DataTransform.cuh:13-46).
class DataTransformer {
public:
    virtual ~DataTransformer() = default;
    virtual int kind() const = 0;  // CRB_NORM_*
    virtual float p0() const = 0;
    virtual float p1() const = 0;
};
class DistribNorm : public DataTransformer {  // (x - mean) * desiredVar / sqrt(var + 1e-8) + desiredMean, per channel
public:
    float desiredMean = 0, desiredVar = 1;
    DistribNorm() = default;
    DistribNorm(float mean, float var) : desiredMean(mean), desiredVar(var) {}
    int kind() const override;
    float p0() const override { return desiredMean; }
    float p1() const override { return desiredVar; }
};
class UniformNorm : public DataTransformer {  // (x - min) / (max - min) * (desiredMax - desiredMin) + desiredMin
public:
    float desiredMin = 0, desiredMax = 1;
    UniformNorm() = default;
    UniformNorm(float min, float max) : desiredMin(min), desiredMax(max) {}
    int kind() const override;
    float p0() const override { return desiredMin; }
    float p1() const override { return desiredMax; }
};

// Augmentations (DataAugmentor.cuh:17-70): each decides per image, when a batch is formed, what the kernel does.
struct ImageAug {  // layout of crb_image_aug
    int32_t dh = 0, dw = 0;
    uint32_t flags = 0;
};
class DataAugmentor {
public:
    uint32 miniBatchSize;
    shape4 dataShape, labelShape;
    DataAugmentor(uint32 miniBatchSize, shape4 dataShape, shape4 labelShape)
        : miniBatchSize(miniBatchSize), dataShape(dataShape), labelShape(labelShape) {}
    virtual ~DataAugmentor() = default;
    virtual void decide(ImageAug &aug, std::default_random_engine &generator) = 0;
};
class RandFlipW : public DataAugmentor {  // mirror along the width with probability 1/2 (DataAugmentor.cu:64-104)
public:
    using DataAugmentor::DataAugmentor;
    void decide(ImageAug &aug, std::default_random_engine &generator) override;
};
class RandCorp : public DataAugmentor {  // shift by offsets uniform in [-pad, pad], zero fill (DataAugmentor.cu:26-62)
public:
    uint32 padH, padW;
    RandCorp(uint32 miniBatchSize, shape4 dataShape, shape4 labelShape, uint32 padH, uint32 padW)
        : DataAugmentor(miniBatchSize, dataShape, labelShape), padH(padH), padW(padW) {}
    void decide(ImageAug &aug, std::default_random_engine &generator) override;
};

// Forms batches of BATCH_SIZE samples as BATCH_SIZE / MINI_BATCH_SIZE mini-batches in device memory, double-buffered
// (Dataset.cuh:17-83, Dataset.cu:20-92): genBatch() fills dataBatch[batchID % 2] and then advances batchID.
struct Dataset {
    Data **dataBatch[2] = {nullptr, nullptr};  // device; views of one buffer per side
    Data **testset = nullptr;                  // device mini-batches filled by allocTestSet()
    uint32 TEST_SIZE = 0;
    DataFetcher *fetcher = nullptr;
    uint32 BATCH_SIZE = 0, EPOCH_SIZE = 0, MAX_EPOCH = 0, MINI_BATCH_SIZE = 0;
    uint32 batchID = 0, epochID = 0;
    shape4 dataShape, labelShape;
    DataTransformer *preProc = nullptr;
    std::vector<DataAugmentor *> augmentations;

    static Dataset *construct(uint32 batchSize, uint32 miniBatchSize, uint32 epochSize, uint32 maxEpoch, shape4 dataShape,
                              shape4 labelShape, uint32 seed = 0);
    void setDataFetcher(DataFetcher *fetch) { fetcher = fetch; }
    void setProcSteps(std::initializer_list<DataTransformer *> steps);  // none or one
    void setAugmentSteps(std::initializer_list<DataAugmentor *> steps);
    void genBatch();
    // TEST_SIZE (the fetcher's) samples drawn by fetchTest, transformed but not augmented, as TEST_SIZE / MINI_BATCH_SIZE
    // device mini-batches in `testset` (Dataset.cu:94-134).
    void allocTestSet();
    std::thread genBatchAsync();
    // What the last genBatch decided per image (for tests and logging).
    const std::vector<ImageAug> &lastAugmentations() const { return augHost; }

private:
    uint8_t *pinnedPixels = nullptr;  // BATCH_SIZE records
    float *pinnedLabels = nullptr;
    ImageAug *pinnedAug = nullptr;
    uint8_t *devPixels = nullptr;
    ImageAug *devAug = nullptr;
    float *devX[2] = {nullptr, nullptr}, *devLabel[2] = {nullptr, nullptr};
    void *stream = nullptr;  // batches are formed on a stream of their own, so that genBatchAsync overlaps training
    std::vector<ImageAug> augHost;
    std::default_random_engine generator;
};
}  // namespace seio
