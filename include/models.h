// xft::Model / xft::AutoModel: a model directory on disk driven to generated token ids.
// Source-compatible with the reference's include/models.h:24-141
//     AutoModel model(path, xft::DataType::int8);
//     model.config(maxLen); model.input(ids, batch);
//     while (!model.isDone()) model.generate();
//     auto out = model.finalize();
// for Llama-family model directories (config.ini + .bin files as the reference's convert tools
// write them, src/models/common_decoder.h:167-262, src/layers/decoder_block.h:205-343) on one
// MI355X.  Served: greedy search, sampling (top-k / top-p / temperature), repetition penalty, stop
// words, beam search, the sequence-id (continuous batching) interface in all nine set_input forms,
// and forward() with the logits of the last or of every position.  Not served: prefix sharing
// (setPrefix / unsetPrefix print a message and exit(-1), the reference's style for an unsupported
// request) and setDecoder (the reference's internal AbstractDecoder has no counterpart here).
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include <cstdint>
#include <string>
#include <tuple>
#include <vector>

#include "abstract_searcher.h"
#include "dtype.h"

namespace xft {

struct ModelImpl; // device model, weights and searcher state (private to the library)

class Model {
public:
    Model();
    ~Model();
    Model(const Model &) = delete;
    Model &operator=(const Model &) = delete;

    // inputIds_: batchSize_ prompts of equal length, row-major (models.cpp:99-115)
    void input(std::vector<int32_t> &inputIds_, int batchSize_);

    void config(int maxLen_ = -1, int numBeams_ = 1, int numBeamHypsToKeep_ = 1, float lenPenalty_ = 1.0,
            bool doEarlyStopping_ = false, int eosTokenId_ = -1, int padTokenId_ = -1, bool doSample_ = false,
            float temperature_ = 1.0, int topK_ = 50, float topP_ = 1.0, float repetitionPenalty_ = 1.0,
            const std::vector<std::vector<int>> &stopWordsList_ = {});

    void config(SearcherConfig &config_, const std::vector<std::vector<int>> &stopWordsList_ = {});

    // Return the sequences' IDs in the order of the input batch
    std::vector<int> set_input(std::vector<int32_t> &inputIds_, int batchSize_, int maxLen_ = -1, int numBeams_ = 1,
            int numBeamHypsToKeep_ = 1, float lenPenalty_ = 1.0, bool doEarlyStopping_ = false, int eosTokenId_ = -1,
            int padTokenId_ = -1, bool doSample_ = false, float temperature_ = 1.0, int topK_ = 50, float topP_ = 1.0,
            float repetitionPenalty_ = 1.0, const std::vector<std::vector<int>> &stopWordsList_ = {});

    // Continuous batching (models.cpp:278-410, 847-903): set_input with no sequence ids turns prompts of any
    // lengths into new sequences and returns their ids; with ids it selects which live sequences the next
    // generate() steps.  generate() runs the prompts (first call) or one decode step, greedy with optional
    // repetition penalty, and marks a sequence done at EOS or at maxLen; finalize() returns the working
    // sequences' tokens back to back and frees them; freeSeqs() frees sequences early.  Every live sequence
    // holds one KV cache row of the device model (8 rows unless XFT_CB_ROWS says otherwise; the model can
    // only grow while no sequence is alive).
    std::vector<int> set_input(std::vector<int32_t> &inputIds_, int batchSize_, SearcherConfig &config_,
            const std::vector<std::vector<int>> &stopWordsList_ = {});

    std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, SearcherConfig &config_,
            const std::vector<std::vector<int>> &stopWordsList_ = {});

    std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, int maxLen_ = -1, int numBeams_ = 1,
            int numBeamHypsToKeep_ = 1, float lenPenalty_ = 1.0, bool doEarlyStopping_ = false, int eosTokenId_ = -1,
            int padTokenId_ = -1, bool doSample_ = false, float temperature_ = 1.0, int topK_ = 50, float topP_ = 1.0,
            float repetitionPenalty_ = 1.0, const std::vector<std::vector<int>> &stopWordsList_ = {});

    std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs,
            SearcherConfig &config_, const std::vector<std::vector<int>> &stopWordsList_ = {});

    // Only used for model.forward(): sequences without a searcher (models.cpp:412-683).  No ids: the prompts
    // become new sequences (maxLen: room to keep for each, -1 / empty = the model's maximum; one value for all
    // or one a sequence).  With ids: inputIds_ holds the next token of every listed sequence, chosen by the caller.
    std::vector<int> set_input(
            std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs = {}, int maxLen = -1);

    // Only used for model.forward()
    std::vector<int> set_input(
            std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs = {}, int maxLen = -1);

    // Only used for model.forward()
    std::vector<int> set_input(
            std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs, const std::vector<int> &maxLen);

    // Only used for model.forward(): prompts of different lengths back to back in inputIds_, their lengths in seqLens_
    std::vector<int> set_input(std::vector<int32_t> &inputIds_, std::vector<int32_t> &seqLens_, std::vector<int> seqIDs,
            std::vector<int> &maxLen);

    bool isDone();

    // After input(): (host pointer to fp32 logits, 0, vocab); the logits of the last position of every
    // sequence [batch, vocab], or of every position [batch * seqLen, vocab] when logitsAll.  After
    // set_input(): (logits, rows, vocab) of the working sequences, all prompts or all decodes; one row a
    // sequence, or one a prompt token when logitsAll and the sequences are prompts (models.cpp:760-830).
    std::tuple<float *, int, int> forward(bool logitsAll = true);

    // One step: the first call after input() runs the prompt, every later call one new token per
    // sequence.  Returns the batch's next token ids (models.cpp:834-846).
    std::vector<int32_t> generate();

    void createSearcher(SearcherConfig &config_);

    bool isMaster() { return true; }

    int getRank() { return 0; }

    int getBatchSize() { return batchSize; }

    int getSeqLen() { return seqLen; }

    void setVocabSize(int vocabSize) { this->vocabSize = vocabSize; }

    int getVocabSize() { return this->vocabSize; }

    void initMaxSeqLen();

    int getMaxSeqLen() { return maxSeqLen; }

    SearcherConfig getConfig() { return configuration; }

    // prompt + generated ids of every sequence, row-major [batch, current length]
    std::vector<int32_t> finalize();

    void exitSlaves() {}

    bool setStopWords(std::vector<std::vector<int>> stopWordsList);

    bool freeSeqs(std::vector<int> &seqIDs);

    // prefix sharing is not served by this build (print + exit(-1))
    void setPrefix(std::vector<int32_t> &prefixIDs);
    void unsetPrefix();

protected:
    ModelImpl *impl;
    std::vector<int32_t> inputIds;
    int batchSize;
    int seqLen;
    int vocabSize;
    int maxSeqLen;
    SearcherConfig configuration;
    bool isNewInput;
};

class AutoModel : public Model {
public:
    AutoModel(std::string modelPath, xft::DataType dataType, xft::DataType KVCacheDataType = xft::DataType::fp16);
};

} // namespace xft
