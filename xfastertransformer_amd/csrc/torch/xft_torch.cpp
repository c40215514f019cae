// torch.classes.xfastertransformer.AutoModel: the Torch custom class the reference's Python package loads
// (src/pytorch/pytorch_warpper.cpp:18-34, src/pytorch/auto_model.h:25-360) with the same method names,
// argument order and tensor conventions (token ids int64 [batch, seq]; logits fp32; sequence ids int64),
// over this library's xft::AutoModel.  Plain g++ against the Torch headers; no HIP here.
#include <torch/custom_class.h>
#include <torch/script.h>

#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/models.h"

namespace {

using OptT = torch::optional<torch::Tensor>;
using OptI = torch::optional<int64_t>;
using OptD = torch::optional<double>;
using OptB = torch::optional<bool>;
using OptWords = torch::optional<std::vector<std::vector<int64_t>>>;

xft::DataType weight_type(const std::string &name) {
    static const std::map<std::string, xft::DataType> names = {{"fp16", xft::DataType::fp16}, {"bf16", xft::DataType::bf16},
            {"int8", xft::DataType::int8}, {"int4", xft::DataType::int4}, {"w8a8", xft::DataType::w8a8}, {"nf4", xft::DataType::nf4},
            {"bf16_fp16", xft::DataType::bf16_fp16}, {"bf16_int8", xft::DataType::bf16_int8}, {"bf16_w8a8", xft::DataType::bf16_w8a8},
            {"bf16_int4", xft::DataType::bf16_int4}, {"bf16_nf4", xft::DataType::bf16_nf4}, {"w8a8_int8", xft::DataType::w8a8_int8},
            {"w8a8_int4", xft::DataType::w8a8_int4}, {"w8a8_nf4", xft::DataType::w8a8_nf4}, {"fp8_e4m3", xft::DataType::fp8_e4m3}};
    auto it = names.find(name);
    if (it == names.end()) throw std::invalid_argument("Invalid data type.");
    return it->second;
}

xft::DataType cache_type(const std::string &name) {
    if (name == "fp16") return xft::DataType::fp16;
    if (name == "bf16") return xft::DataType::bf16;
    if (name == "int8") return xft::DataType::int8;
    throw std::invalid_argument("Invalid KV cache data type.");
}

// every element of an integer tensor of any shape, in memory order, as int
std::vector<int> ints_of(const torch::Tensor &t) {
    const torch::Tensor flat = t.to(torch::kCPU, torch::kInt64).contiguous();
    const int64_t *p = flat.data_ptr<int64_t>();
    return std::vector<int>(p, p + flat.numel());
}

torch::Tensor int64_tensor(const std::vector<int> &v, std::vector<int64_t> shape) {
    torch::Tensor out = torch::empty(shape, torch::kInt64);
    TORCH_CHECK((size_t)out.numel() == v.size(), "internal: ", v.size(), " values for a tensor of ", out.numel());
    int64_t *p = out.data_ptr<int64_t>();
    for (size_t i = 0; i < v.size(); ++i) p[i] = v[i];
    return out;
}

struct Generation {
    SearcherConfig config;
    std::vector<std::vector<int>> stopWords;
};

Generation generation_of(OptI maxLength, OptI numBeams, OptI numReturnSequences, OptD lenPenalty, OptB earlyStopping, OptI eosTokenId,
        OptI padTokenId, OptB doSample, OptD temperature, OptI topK, OptD topP, OptD repetitionPenalty, const OptWords &stopWordsList) {
    TORCH_CHECK(maxLength.has_value(), "Make sure master's maxLen is not None.")
    Generation g;
    g.config.maxLen = (int)maxLength.value();
    g.config.numBeams = (int)numBeams.value_or(1);
    g.config.numBeamHypsToKeep = (int)numReturnSequences.value_or(1);
    g.config.lenPenalty = (float)lenPenalty.value_or(1.0);
    g.config.doEarlyStopping = earlyStopping.value_or(false);
    g.config.eosTokenId = (int)eosTokenId.value_or(-1);
    g.config.padTokenId = (int)padTokenId.value_or(-1);
    g.config.doSample = doSample.value_or(false);
    g.config.temperature = (float)temperature.value_or(1.0);
    g.config.topK = (int)topK.value_or(50);
    g.config.topP = (float)topP.value_or(1.0);
    g.config.repetitionPenalty = (float)repetitionPenalty.value_or(1.0);
    if (stopWordsList.has_value())
        for (const auto &word : stopWordsList.value()) g.stopWords.emplace_back(word.begin(), word.end());
    return g;
}

} // namespace

struct TorchAutoModel : torch::CustomClassHolder {
    TorchAutoModel(std::string modelPath, std::string dtype, std::string KVCacheDtype)
        : model(modelPath, weight_type(dtype), cache_type(KVCacheDtype)) {}

    int64_t getRank() { return model.getRank(); }

    bool isDone() { return model.isDone(); }

    void input(OptT inputIds) {
        TORCH_CHECK(inputIds.has_value(), "Make sure master's input is not None.")
        TORCH_CHECK(inputIds.value().dim() == 2, "input ids must be [batch, seqLen]")
        ids = ints_of(inputIds.value());
        model.input(ids, (int)inputIds.value().size(0));
    }

    void config(OptI maxLength, OptI numBeams, OptI numReturnSequences, OptD lenPenalty, OptB earlyStopping, OptI eosTokenId, OptI padTokenId,
            OptB doSample, OptD temperature, OptI topK, OptD topP, OptD repetitionPenalty, OptWords stopWordsList) {
        Generation g = generation_of(maxLength, numBeams, numReturnSequences, lenPenalty, earlyStopping, eosTokenId, padTokenId, doSample,
                temperature, topK, topP, repetitionPenalty, stopWordsList);
        model.config(g.config, g.stopWords);
    }

    // new sequences with their searcher configuration (the caller then drives generate())
    void setInput(OptT inputIds, OptI maxLength, OptI numBeams, OptI numReturnSequences, OptD lenPenalty, OptB earlyStopping, OptI eosTokenId,
            OptI padTokenId, OptB doSample, OptD temperature, OptI topK, OptD topP, OptD repetitionPenalty, OptWords stopWordsList) {
        Generation g = generation_of(maxLength, numBeams, numReturnSequences, lenPenalty, earlyStopping, eosTokenId, padTokenId, doSample,
                temperature, topK, topP, repetitionPenalty, stopWordsList);
        TORCH_CHECK(inputIds.has_value(), "Make sure master's input is not None.")
        TORCH_CHECK(inputIds.value().dim() == 2, "input ids must be [batch, seqLen]")
        ids = ints_of(inputIds.value());
        model.set_input(ids, (int)inputIds.value().size(0), g.config, g.stopWords);
    }

    // logits of every position of a batch of prompts: [batch, seqLen, vocab] over memory the model owns
    torch::Tensor forward(torch::Tensor &inputIds) {
        input(inputIds);
        float *logits = std::get<0>(model.forward());
        return torch::from_blob(logits, {inputIds.size(0), inputIds.size(1), (int64_t)model.getVocabSize()}, torch::kFloat32);
    }

    torch::Tensor generate() {
        const std::vector<int32_t> next = model.generate();
        return int64_tensor(std::vector<int>(next.begin(), next.end()), {(int64_t)model.getBatchSize(), (int64_t)model.getConfig().numBeams});
    }

    torch::Tensor finalize() {
        const std::vector<int32_t> out = model.finalize();
        const int64_t rows = (int64_t)model.getBatchSize() * model.getConfig().numBeamHypsToKeep;
        TORCH_CHECK(rows > 0 && out.size() % (size_t)rows == 0, "finalize: ", out.size(), " ids do not form ", rows, " rows")
        return int64_tensor(std::vector<int>(out.begin(), out.end()), {rows, (int64_t)(out.size() / (size_t)rows)});
    }

    void setPrefix(OptT inputIds) {
        TORCH_CHECK(inputIds.has_value(), "Make sure master's prefix input is not None.")
        TORCH_CHECK(inputIds.value().dim() <= 2, "Prefix sharing input expected dim <= 2 but tensor has ", inputIds.value().dim());
        TORCH_CHECK(inputIds.value().dim() == 1 || inputIds.value().size(0) == 1, "Prefix sharing only support 1 prompt but input has ",
                inputIds.value().size(0));
        std::vector<int> prefix = ints_of(inputIds.value());
        model.setPrefix(prefix);
    }

    void unsetPrefix() { model.unsetPrefix(); }

    // one pass of the sequences chosen by set_input_cb: [sequences, vocab], the last position of each
    torch::Tensor forwardCB() {
        const std::tuple<float *, int, int> r = model.forward(false);
        return torch::from_blob(std::get<0>(r), {(int64_t)std::get<1>(r), (int64_t)std::get<2>(r)}, torch::kFloat32);
    }

    // 2-D ids: prompts of one length (no seqIDs) or the next token of each listed sequence ([batch, 1] with seqIDs);
    // 1-D ids: prompts of different lengths back to back, their lengths in seqLens.  Returns the sequence ids.
    torch::Tensor setInputCB(OptT inputIds, OptT seqLens, OptT seqIDs, OptT maxLens) {
        TORCH_CHECK(inputIds.has_value(), "Make sure master's input is not None.")
        const torch::Tensor &t = inputIds.value();
        TORCH_CHECK(t.dim() == 2 || t.dim() == 1, "Make sure master's input is 1-D or 2-D.")
        std::vector<int> lens, seqs, maxs;
        int64_t batch;
        if (t.dim() == 2) {
            batch = t.size(0);
            lens.assign((size_t)batch, (int)t.size(1));
        } else {
            TORCH_CHECK(seqLens.has_value(), "Make sure master's seqLens_ is not None when input is 1-D.")
            TORCH_CHECK(seqLens.value().dim() == 1, "Make sure master's seqLens_ is 1-D.")
            TORCH_CHECK(!seqIDs.has_value(), "Make sure master's seqIDs_ is None when input is 1-D.")
            lens = ints_of(seqLens.value());
            batch = (int64_t)lens.size();
        }
        ids = ints_of(t);
        if (seqIDs.has_value()) {
            seqs = ints_of(seqIDs.value());
            TORCH_CHECK((int64_t)seqs.size() == batch, "seqIDs'shape must equal to batchSize.")
        }
        if (maxLens.has_value()) {
            maxs = ints_of(maxLens.value());
            TORCH_CHECK((int64_t)maxs.size() == batch || maxs.size() == 1, "maxLens size must equal to inputIds size[0] or 1.")
        }
        const std::vector<int> out = model.set_input(ids, lens, seqs, maxs);
        return int64_tensor(out, {(int64_t)out.size()});
    }

    bool freeSeqs(OptT seqIDs) {
        TORCH_CHECK(seqIDs.has_value(), "Make sure master's input is not None.")
        std::vector<int> seqs = ints_of(seqIDs.value());
        return model.freeSeqs(seqs);
    }

private:
    xft::AutoModel model;
    std::vector<int> ids; // the model keeps references to its input for the length of a call only; kept for input()
};

TORCH_LIBRARY(xfastertransformer, m) {
    m.class_<TorchAutoModel>("AutoModel")
            .def(torch::init<std::string, std::string, std::string>())
            .def("get_rank", &TorchAutoModel::getRank)
            .def("input", &TorchAutoModel::input)
            .def("config", &TorchAutoModel::config)
            .def("set_input", &TorchAutoModel::setInput)
            .def("set_input_cb", &TorchAutoModel::setInputCB)
            .def("is_done", &TorchAutoModel::isDone)
            .def("forward", &TorchAutoModel::forward)
            .def("forward_cb", &TorchAutoModel::forwardCB)
            .def("generate", &TorchAutoModel::generate)
            .def("finalize", &TorchAutoModel::finalize)
            .def("free_seqs", &TorchAutoModel::freeSeqs)
            .def("set_prefix", &TorchAutoModel::setPrefix)
            .def("unset_prefix", &TorchAutoModel::unsetPrefix);
}
