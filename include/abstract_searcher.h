// Generation settings of xft::Model (source-compatible with the field names, order and defaults
// of the reference's include/abstract_searcher.h:38-67).
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

struct SearcherConfig {
    bool doEarlyStopping = false;
    bool doSample = false;
    int maxLen = -1;
    int numBeams = 1;
    int numBeamHypsToKeep = 1;
    int eosTokenId = -1;
    int padTokenId = -1;
    int topK = 50;
    float lenPenalty = 1.0;
    float temperature = 1.0;
    float topP = 1.0;
    float repetitionPenalty = 1.0;

    SearcherConfig(int maxLen_ = -1, int numBeams_ = 1, int numBeamHypsToKeep_ = 1, float lenPenalty_ = 1.0,
            bool doEarlyStopping_ = false, int eosTokenId_ = -1, int padTokenId_ = -1, bool doSample_ = false,
            float temperature_ = 1.0, int topK_ = 50, float topP_ = 1.0, float repetitionPenalty_ = 1.0)
        : doEarlyStopping(doEarlyStopping_)
        , doSample(doSample_)
        , maxLen(maxLen_)
        , numBeams(numBeams_)
        , numBeamHypsToKeep(numBeamHypsToKeep_)
        , eosTokenId(eosTokenId_)
        , padTokenId(padTokenId_)
        , topK(topK_)
        , lenPenalty(lenPenalty_)
        , temperature(temperature_)
        , topP(topP_)
        , repetitionPenalty(repetitionPenalty_) {}
};
