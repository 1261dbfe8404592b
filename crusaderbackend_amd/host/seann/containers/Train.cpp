// Sequential::train — kept in a translation unit of its own because it joins the network container with the seio data
// pipeline and model files.
#include <cstdio>
#include <fstream>
#include <stdexcept>
#include <string>

#include "../../seio/data/Dataset.h"
#include "../../seio/modelcache/codec.h"
#include "Sequential.h"

namespace seann {

void Sequential::train(seio::Dataset *data, bool WITH_TEST, uint32 TEST_FREQUENCY, const char *cacheDir, TrainProgress progress) {
    if (!data || !data->BATCH_SIZE || data->MINI_BATCH_SIZE != netX->A->dims.n)
        throw std::invalid_argument("Sequential::train: the dataset's mini-batch size must be the network's batch size");
    if (!loss || !lossFW) throw std::invalid_argument("Sequential::train: no loss function set");
    if (WITH_TEST && (!data->testset || !TEST_FREQUENCY)) throw std::invalid_argument("Sequential::train: no test set allocated");
    const std::string dir = std::string(cacheDir) + "/";
    data->genBatch();
    Tensor *lossBuf = Tensor::create(netY->A->dims);
    std::remove((dir + "cache.log").c_str());
    std::fstream trainLog(dir + "cache.log", std::ios::binary | std::ios::out);
    const uint32 minis = data->BATCH_SIZE / data->MINI_BATCH_SIZE;
    while (data->epochID < data->MAX_EPOCH) {
        const uint32 batchID = data->batchID - 1, epochID = data->epochID;
        std::thread pass = data->genBatchAsync();
        float batchLoss = 0;
        try {
            for (uint32 sampleID = 0; sampleID < minis; sampleID++) {
                seio::Data *mb = data->dataBatch[batchID % 2][sampleID];
                forward(mb->X);
                backward(mb->label);
                batchLoss += lossFW(netY, mb->label, lossBuf);
                learn();
            }
            learnBatch();
        } catch (...) {
            pass.join();
            throw;
        }
        trainLog << batchLoss / float(data->BATCH_SIZE) << ", ";
        pass.join();  // the next batch is in place

        float lossVal = 0;
        if (WITH_TEST && data->batchID % TEST_FREQUENCY == 0) {
            for (uint32 i = 0; i < data->TEST_SIZE / data->MINI_BATCH_SIZE; i++) {
                inferenceForward(data->testset[i]->X);
                lossVal += lossFW(netY, data->testset[i]->label, lossBuf);
            }
            lossVal /= float(data->TEST_SIZE);
            trainLog << lossVal << ",";
        }
        if (data->epochID != epochID) {
            zeroGrads();
            if (epochID % 5 == 0) {
                std::remove((dir + "cache.crseq").c_str());
                seio::saveSequence((dir + "cache.crseq").c_str(), this, epochID);
            }
        }
        if (progress) progress(epochID, batchID, batchLoss / float(data->BATCH_SIZE), lossVal);
    }
    trainLog.close();
    lossBuf->eliminate();
}
}  // namespace seann
