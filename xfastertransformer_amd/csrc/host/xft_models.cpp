// xft::Model / xft::AutoModel over the C-ABI of the gfx950 library: the on-disk model format of the
// reference (config.ini + one .bin per tensor) loaded into a device-resident decoder stack, and
// the searchers that turn its logits into token ids.
//
// Replaces, for Llama-family directories on one GPU:
//   AutoModel::AutoModel / Model::input / config / generate / isDone / finalize (src/models/models.cpp:99-135,
//   706-758, 834-846, 1014-1035), CommonDecoder's constructor (src/models/common_decoder.h:167-262: the
//   config.ini keys), DecoderBlock's weight loading (src/layers/decoder_block.h:205-343: the file names and
//   shapes), CommonDecoder::setEmbeddingWeights / setFinalLnWeight / setPredictorWeight
//   (common_decoder.h:857-874, llama.cpp:46-51), GreedySearch and SampleSearch
//   (src/searchers/greedy_search.cpp, sample_search.cpp) and the repetition penalty / stop-word helpers
//   (src/searchers/search_utils.cpp:22-99).
// Plain C++ (g++), no HIP headers.  Failures print a message and exit(-1), as the reference does.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <random>
#include <set>
#include <limits>
#include <string>
#include <tuple>
#include <vector>

#include "../../../include/models.h"
#include "../../../include/xft_hip.h"
#include "host_util.h"

using namespace xfthost;

namespace {

// ---- config.ini ---------------------------------------------------------------------------------
// Section / key lookup is case-insensitive and the "first" section is the smallest name of an ordered
// set, the behaviour of the INIReader the reference uses (models.cpp:1023: *reader.Sections().begin()).
struct Ini {
    std::set<std::string> sections;
    std::map<std::string, std::string> values;
    bool ok = false;

    static std::string lower(std::string s) {
        for (auto &c : s) c = (char)tolower((unsigned char)c);
        return s;
    }
    static std::string trim(const std::string &s) {
        size_t a = 0, b = s.size();
        while (a < b && isspace((unsigned char)s[a])) ++a;
        while (b > a && isspace((unsigned char)s[b - 1])) --b;
        return s.substr(a, b - a);
    }
    explicit Ini(const std::string &path) {
        FILE *f = fopen(path.c_str(), "r");
        if (!f) return;
        ok = true;
        char line[4096];
        std::string section;
        while (fgets(line, sizeof(line), f)) {
            std::string s = trim(line);
            if (s.empty() || s[0] == ';' || s[0] == '#') continue;
            if (s[0] == '[') {
                const size_t e = s.find(']');
                if (e == std::string::npos) continue;
                section = trim(s.substr(1, e - 1));
                sections.insert(section);
                continue;
            }
            size_t eq = s.find_first_of("=:");
            if (eq == std::string::npos) continue;
            std::string key = trim(s.substr(0, eq)), val = trim(s.substr(eq + 1));
            // an inline comment starts at " ;" or " #"
            for (size_t i = 1; i < val.size(); ++i)
                if ((val[i] == ';' || val[i] == '#') && isspace((unsigned char)val[i - 1])) {
                    val = trim(val.substr(0, i));
                    break;
                }
            values[lower(section) + "=" + lower(key)] = val;
        }
        fclose(f);
    }
    bool has(const std::string &sec, const std::string &key) const { return values.count(lower(sec) + "=" + lower(key)) != 0; }
    std::string get(const std::string &sec, const std::string &key, const std::string &dflt = "") const {
        auto it = values.find(lower(sec) + "=" + lower(key));
        return it == values.end() ? dflt : it->second;
    }
    long get_int(const std::string &sec, const std::string &key, long dflt) const {
        const std::string v = get(sec, key);
        if (v.empty()) return dflt;
        char *end = nullptr;
        const long r = strtol(v.c_str(), &end, 0);
        return end > v.c_str() ? r : dflt;
    }
    double get_float(const std::string &sec, const std::string &key, double dflt) const {
        const std::string v = get(sec, key);
        if (v.empty()) return dflt;
        char *end = nullptr;
        const double r = strtod(v.c_str(), &end);
        return end > v.c_str() ? r : dflt;
    }
};

bool file_exists(const std::string &p) {
    FILE *f = fopen(p.c_str(), "rb");
    if (!f) return false;
    fclose(f);
    return true;
}

// Reads `count` elements of `wtype` (fp32 / fp16 / bf16 as config.ini's weight_data_type names it,
// src/utils/weight_util.h:37-67, 139-167) and widens them to fp32.  A missing optional file gives an
// empty vector; a short or missing required file ends the process.
std::vector<float> read_floats(const std::string &path, size_t count, xft::DataType wtype, bool required = true) {
    std::vector<float> out;
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) {
        if (required) {
            printf("Cannot open the weight file %s\n", path.c_str());
            exit(-1);
        }
        return out;
    }
    out.resize(count);
    size_t got = 0;
    if (wtype == xft::DataType::fp32) {
        got = fread(out.data(), 4, count, f);
    } else {
        std::vector<uint16_t> raw(count);
        got = fread(raw.data(), 2, count, f);
        if (wtype == xft::DataType::fp16)
            for (size_t i = 0; i < got; ++i) out[i] = from_fp16(raw[i]);
        else
            for (size_t i = 0; i < got; ++i) out[i] = from_bf16(raw[i]);
    }
    fclose(f);
    if (got != count) {
        printf("Weight file %s holds %zu elements, %zu expected\n", path.c_str(), got, count);
        exit(-1);
    }
    return out;
}

std::vector<uint8_t> read_bytes(const std::string &path, size_t count) {
    std::vector<uint8_t> out(count);
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) {
        printf("Cannot open the weight file %s\n", path.c_str());
        exit(-1);
    }
    const size_t got = fread(out.data(), 1, count, f);
    fclose(f);
    if (got != count) {
        printf("Weight file %s holds %zu bytes, %zu expected\n", path.c_str(), got, count);
        exit(-1);
    }
    return out;
}

const char *type_name(xft::DataType dt) {
    switch (dt) {
        case xft::DataType::fp32: return "fp32";
        case xft::DataType::bf16: return "bf16";
        case xft::DataType::fp16: return "fp16";
        case xft::DataType::int8: return "int8";
        case xft::DataType::w8a8: return "w8a8";
        case xft::DataType::int4: return "int4";
        case xft::DataType::nf4: return "nf4";
        case xft::DataType::bf16_fp16: return "bf16_fp16";
        case xft::DataType::bf16_int8: return "bf16_int8";
        case xft::DataType::bf16_w8a8: return "bf16_w8a8";
        case xft::DataType::bf16_int4: return "bf16_int4";
        case xft::DataType::bf16_nf4: return "bf16_nf4";
        case xft::DataType::w8a8_int8: return "w8a8_int8";
        case xft::DataType::w8a8_int4: return "w8a8_int4";
        case xft::DataType::w8a8_nf4: return "w8a8_nf4";
        case xft::DataType::fp8_e4m3: return "fp8_e4m3";
        default: return "unknown";
    }
}

// One [K, N] matrix of the directory, in whichever form the files hold it.
struct HostMatrix {
    int K = 0, N = 0;
    std::vector<float> w; // fp32 [K, N] (plain files)
    int qkind = -1; // XFTHIP_W_INT8 / XFTHIP_W_UINT4 when the directory is pre-quantised
    std::vector<uint8_t> q;
    std::vector<float> scale, zero;
};

// horizontal concatenation of matrices with the same K: [K, sum N]
HostMatrix hcat(const std::vector<const HostMatrix *> &parts) {
    HostMatrix out;
    out.K = parts[0]->K;
    out.qkind = parts[0]->qkind;
    for (auto *p : parts) out.N += p->N;
    if (out.qkind < 0) {
        out.w.resize((size_t)out.K * out.N);
        int off = 0;
        for (auto *p : parts) {
            for (int k = 0; k < out.K; ++k) memcpy(&out.w[(size_t)k * out.N + off], &p->w[(size_t)k * p->N], sizeof(float) * p->N);
            off += p->N;
        }
        return out;
    }
    const int per = out.qkind == XFTHIP_W_UINT4 ? 2 : 1; // columns per byte
    out.q.resize((size_t)out.K * out.N / per);
    int off = 0;
    for (auto *p : parts) {
        for (int k = 0; k < out.K; ++k)
            memcpy(&out.q[((size_t)k * out.N + off) / per], &p->q[(size_t)k * p->N / per], (size_t)p->N / per);
        out.scale.insert(out.scale.end(), p->scale.begin(), p->scale.end());
        out.zero.insert(out.zero.end(), p->zero.begin(), p->zero.end());
        off += p->N;
    }
    return out;
}

} // namespace

namespace xft {

// ---- beam search: the host half (reference src/searchers/beam_search.cpp) --------------------------
// One object holds what BeamSearch, BeamSearchScorer and BeamHypotheses hold there.  The device supplies
// the logits of every beam row and copies cache rows; everything else is integer / float bookkeeping.
struct BeamSearcher {
    struct Hyps { // BeamHypotheses (:86-116)
        std::vector<std::pair<float, std::vector<int32_t>>> beams;
        float worst = 1e9f;
    };
    int batch = 0, numBeams = 0, keep = 1, maxLen = 0, kVal = 0, vocab = 0, eos = -1, pad = -1;
    float lenPenalty = 1.0f;
    bool early = false;
    std::vector<Hyps> hyps;
    std::vector<char> done;
    std::vector<int32_t> inputIds; // [batch * numBeams][len]
    int len = 0; // tokens of a row of inputIds
    std::vector<float> beamScores;
    std::vector<int> beamTokens, beamIndices;
    int steps = 0;

    int rows() const { return batch * numBeams; }

    void start(const int32_t *ids, int batch_, int seqLen, int numBeams_, int keep_, int maxLen_, float lenPenalty_, bool early_, int eos_,
            int pad_, int vocab_) {
        batch = batch_, numBeams = numBeams_, keep = keep_, maxLen = maxLen_, lenPenalty = lenPenalty_, early = early_;
        eos = eos_, pad = pad_, vocab = vocab_, kVal = 2 * numBeams_, steps = 0;
        if (numBeams <= 1) {
            printf("numBeams has to be an integer strictly greater than 1\n");
            exit(-1);
        }
        hyps.assign(batch, Hyps());
        done.assign(batch, 0);
        len = seqLen;
        inputIds.resize((size_t)rows() * seqLen);
        for (int b = 0; b < batch; ++b)
            for (int j = 0; j < numBeams; ++j)
                std::copy(ids + (size_t)b * seqLen, ids + (size_t)(b + 1) * seqLen, inputIds.begin() + ((size_t)b * numBeams + j) * seqLen);
        // all candidates of the first step come from beam 0 (:296-300)
        beamScores.assign(rows(), -1e9f);
        for (int b = 0; b < batch; ++b) beamScores[(size_t)b * numBeams] = 0.0f;
        beamTokens.assign(rows(), 0);
        beamIndices.assign(rows(), 0);
    }

    void add_hyp(Hyps &h, std::vector<int32_t> hyp, float sumLogProbs) const { // :89-104
        const float score = sumLogProbs / std::pow((float)hyp.size(), lenPenalty);
        if ((int)h.beams.size() < numBeams || score > h.worst) {
            h.beams.emplace_back(score, std::move(hyp));
            if ((int)h.beams.size() > numBeams) {
                std::sort(h.beams.begin(), h.beams.end(), [](const auto &a, const auto &b) { return a.first < b.first; });
                h.beams.erase(h.beams.begin());
                h.worst = h.beams[0].first;
            } else {
                h.worst = std::min(score, h.worst);
            }
        }
    }

    bool hyps_done(const Hyps &h, float bestSumLogProbs, int curLen) const { // :106-116
        if ((int)h.beams.size() < numBeams) return false;
        if (early) return true;
        return h.worst >= bestSumLogProbs / std::pow((float)curLen, lenPenalty);
    }

    bool all_done() const {
        for (char f : done)
            if (!f) return false;
        return true;
    }

    // logits: fp32 [rows][vocab], overwritten by their log-softmax.  Chooses the next token and the
    // source row of every beam row (searchTopK + BeamSearchScorer::process + the inputIds update).
    void step(float *logits) {
        const int R = rows();
        std::vector<float> topVals((size_t)R * kVal);
        std::vector<int> topIds((size_t)R * kVal);
        for (int i = 0; i < R; ++i) {
            float *p = logits + (size_t)i * vocab;
            float mx = std::numeric_limits<float>::lowest();
            for (int j = 0; j < vocab; ++j) mx = std::max(mx, p[j]);
            float sum = 0.0f;
            for (int j = 0; j < vocab; ++j) sum += std::exp(p[j] - mx);
            const float sub = mx + std::log(sum);
            for (int j = 0; j < vocab; ++j) p[j] -= sub;
            // the kVal largest in the order of std::greater<std::pair<float, int>> (:470-481)
            std::vector<std::pair<float, int>> best;
            best.reserve(kVal + 1);
            for (int j = 0; j < vocab; ++j) {
                const std::pair<float, int> e(p[j], j);
                if ((int)best.size() == kVal && !(e > best.back())) continue;
                best.insert(std::upper_bound(best.begin(), best.end(), e, std::greater<std::pair<float, int>>()), e);
                if ((int)best.size() > kVal) best.pop_back();
            }
            for (int j = 0; j < kVal; ++j) {
                topVals[(size_t)i * kVal + j] = best[j].first + beamScores[i];
                topIds[(size_t)i * kVal + j] = best[j].second;
            }
        }
        // per user sequence: the kVal best of its beams' candidates, equal (score, token) pairs once (:528-547)
        std::vector<float> nextScores((size_t)batch * kVal);
        std::vector<int> nextTokens((size_t)batch * kVal), nextIndices((size_t)batch * kVal);
        for (int b = 0; b < batch; ++b) {
            std::vector<std::tuple<float, int, int>> el((size_t)numBeams * kVal);
            for (int j = 0; j < numBeams; ++j)
                for (int k = 0; k < kVal; ++k) {
                    const size_t at = ((size_t)b * numBeams + j) * kVal + k;
                    el[(size_t)j * kVal + k] = std::make_tuple(topVals[at], topIds[at], j);
                }
            std::stable_sort(el.begin(), el.end(), [](const auto &x, const auto &y) {
                if (std::get<0>(x) > std::get<0>(y)) return true;
                return std::get<0>(x) == std::get<0>(y) && std::get<2>(x) < std::get<2>(y);
            });
            (void)std::unique(el.begin(), el.end(),
                    [](const auto &x, const auto &y) { return std::get<0>(x) == std::get<0>(y) && std::get<1>(x) == std::get<1>(y); });
            for (int k = 0; k < kVal; ++k) {
                nextScores[(size_t)b * kVal + k] = std::get<0>(el[k]);
                nextTokens[(size_t)b * kVal + k] = std::get<1>(el[k]);
                nextIndices[(size_t)b * kVal + k] = std::get<2>(el[k]);
            }
        }
        // BeamSearchScorer::process (:137-193): len is still the length before this step's token
        std::vector<float> newScores(R, 0.0f);
        std::vector<int> newTokens(R, pad), newIndices(R, 0);
        for (int b = 0; b < batch; ++b) {
            if (done[b]) continue; // its rows are fed the pad token from row 0
            int beamIdx = 0;
            for (int rank = 0; rank < kVal; ++rank) {
                const int tok = nextTokens[(size_t)b * kVal + rank];
                const float sc = nextScores[(size_t)b * kVal + rank];
                const int row = b * numBeams + nextIndices[(size_t)b * kVal + rank];
                if (eos != -1 && tok == eos) {
                    if (rank >= numBeams) continue;
                    add_hyp(hyps[b], std::vector<int32_t>(inputIds.begin() + (size_t)row * len, inputIds.begin() + (size_t)(row + 1) * len), sc);
                } else {
                    newScores[(size_t)b * numBeams + beamIdx] = sc;
                    newTokens[(size_t)b * numBeams + beamIdx] = tok;
                    newIndices[(size_t)b * numBeams + beamIdx] = row;
                    if (++beamIdx == numBeams) break;
                }
            }
            if (beamIdx < numBeams) {
                printf("At most tokens can be equal to `eosTokenId`\n");
                exit(-1);
            }
            // the reference takes this maximum over nextScores[b * numBeams .. (b + 1) * numBeams), although a
            // user sequence owns kVal = 2 * numBeams entries (:187-190); kept as it is
            const float best = *std::max_element(nextScores.begin() + (size_t)b * numBeams, nextScores.begin() + (size_t)(b + 1) * numBeams);
            done[b] = done[b] || hyps_done(hyps[b], best, len);
        }
        beamScores = newScores, beamTokens = newTokens, beamIndices = newIndices;
        // every row continues the history of its source row (:553-563)
        std::vector<int32_t> grown((size_t)R * (len + 1));
        for (int i = 0; i < R; ++i) {
            std::copy(inputIds.begin() + (size_t)beamIndices[i] * len, inputIds.begin() + (size_t)(beamIndices[i] + 1) * len,
                    grown.begin() + (size_t)i * (len + 1));
            grown[(size_t)(i + 1) * (len + 1) - 1] = beamTokens[i];
        }
        inputIds.swap(grown);
        ++len;
        ++steps;
    }

    bool is_done() const { return steps != 0 && (all_done() || len >= maxLen); } // :330-332

    std::vector<int32_t> finalize() { // BeamSearchScorer::finalize (:195-263)
        for (int b = 0; b < batch; ++b) {
            if (done[b]) continue;
            for (int j = 0; j < numBeams; ++j) {
                const size_t row = (size_t)b * numBeams + j;
                add_hyp(hyps[b], std::vector<int32_t>(inputIds.begin() + row * len, inputIds.begin() + (row + 1) * len), beamScores[row]);
            }
        }
        std::vector<std::vector<int32_t>> best;
        std::vector<int> lens;
        for (int b = 0; b < batch; ++b) {
            auto sorted = hyps[b].beams;
            std::sort(sorted.begin(), sorted.end(), [](const auto &x, const auto &y) { return x.first < y.first; });
            for (int j = 0; j < keep; ++j) {
                if (sorted.empty()) {
                    printf("numBeamHypsToKeep (%d) exceeds the hypotheses kept for a sequence.\n", keep);
                    exit(-1);
                }
                best.push_back(sorted.back().second);
                lens.push_back((int)sorted.back().second.size());
                sorted.pop_back();
            }
        }
        const int longest = *std::max_element(lens.begin(), lens.end());
        const int outLen = std::min(longest + 1, maxLen);
        std::vector<int32_t> decoded((size_t)best.size() * outLen, pad);
        for (size_t i = 0; i < best.size(); ++i) {
            if (lens[i] < maxLen) {
                std::copy(best[i].begin(), best[i].end(), decoded.begin() + i * outLen);
                decoded[i * outLen + lens[i]] = eos;
            } else {
                std::copy(best[i].begin(), best[i].begin() + maxLen, decoded.begin() + i * outLen);
            }
        }
        return decoded;
    }
};

struct ModelImpl {
    std::string path, modelType;
    xft::DataType fileType = xft::DataType::fp32;
    int fileQuant = -1; // weight kind of pre-quantised files or -1
    int wkind = XFTHIP_W_BF16;
    int firstKind = -1; // weight kind of the prompt pass when it differs (the mixed "first_next" types), else -1
    int kvDtype = XFTHIP_FP16;
    int layers = 0, hidden = 0, inter = 0, heads = 0, kvHeads = 0, headSize = 0, vocab = 0;
    int maxPosEmbed = 0, maxPositions = 0, maxSeqLength = -1, startId = 0, endId = 0;
    float eps = 1e-6f, ropeTheta = 10000.0f;

    struct Layer {
        xfthip_weight_t qkv = nullptr, o = nullptr, gateup = nullptr, down = nullptr;
        xfthip_weight_t firstQkv = nullptr, firstO = nullptr, firstGateup = nullptr, firstDown = nullptr;
        std::vector<float> ln1, ln2, qkvBias, oBias;
        // [mixtral] directories: the router [hidden, experts] and every expert's gate/up and down weights
        // (MixtralFFNParams, decoder_block.h:640-676); gateup / down above stay empty
        std::vector<float> router;
        std::vector<xfthip_weight_t> expertGateup, expertDown;
    };
    // prefix sharing (Model::setPrefix): the prefix ids, and whether the device model's cache row 0 holds them
    std::vector<int32_t> prefix;
    bool prefixOnDevice = false;
    int experts = 0; // sparse_experts of a [mixtral] section, 0 for a dense model
    std::vector<xfthip_moe_t> moe; // one per layer, rebuilt with the device model (their buffers are sized by its token capacity)
    std::vector<Layer> L;
    std::vector<uint16_t> embedding;
    std::vector<float> finalNorm;
    xfthip_weight_t lmHead = nullptr;
    size_t weightBytes = 0;

    xfthip_model_t model = nullptr;
    xfthip_model_config cfg {};

    // searcher state (GreedySearch / SampleSearch members of the reference)
    bool haveSearcher = false, sampling = false;
    int maxLen = 0, eosTokenId = -1, padTokenId = -1, topK = 50;
    float topP = 1.0f, temperatureInv = 1.0f, repetitionPenalty = 1.0f;
    std::vector<std::vector<int>> stopWordsList, stopWordsIndex, cachedRepetVec;
    std::vector<int> doneBatch, nextTokens, deviceIds;
    std::vector<int32_t> output;
    std::vector<float> logitsHost;
    int step = 0, curLen = 0, batch = 0;
    std::mt19937_64 rng {std::random_device {}()};
    bool beam = false; // numBeams > 1: BeamSearch instead of Greedy / SampleSearch
    int numBeams = 1, numBeamHypsToKeep = 1;
    float lenPenalty = 1.0f;
    bool doEarlyStopping = false;
    BeamSearcher beams;

    // continuous batching (Model::set_input / generate / freeSeqs): the sequence pool and the
    // sequence-id -> cache-row map, the roles of SequencePool and KVCacheMgr
    // (src/common/sequence.h, src/common/kvcache_mgr.h:37-194)
    struct Seq {
        int id = 0, row = 0, step = 0;
        bool done = false;
        bool forwardOnly = false; // made by the set_input forms that carry no searcher config: Model::forward() runs it
        std::vector<int32_t> prompt, generated;
        SearcherConfig cfg;
        std::vector<int> cachedRepetVec;
    };
    std::map<int, Seq> pool;
    std::vector<int> working; // ids of the sequences the next generate() call steps
    int nextSeqId = 0;
    bool cbMode = false;

    int free_row() const {
        std::vector<char> used(cfg.max_batch, 0);
        for (auto &kv : pool) used[kv.second.row] = 1;
        for (int r = 0; r < cfg.max_batch; ++r)
            if (!used[r]) return r;
        return -1;
    }

    // Room for `add` more sequences of up to maxLen tokens.  The device model (and with it every cache row)
    // is rebuilt when it has to grow, which is only possible while no sequence is alive.
    void fit_rows(int add, int maxLen, int longestPrompt) {
        const int live = (int)pool.size();
        // Cache rows the pool starts with: XFT_CB_ROWS, or as many rows of maxLen + 1 positions as fit 40 % of the free
        // device memory, between 8 and 64 (a row is layers x 2 x kv heads x positions x head size values of the cache's
        // type; the weights are already on the device when the pool is sized)
        int rows = 8;
        if (const char *e = getenv("XFT_CB_ROWS")) {
            rows = atoi(e) > 0 ? atoi(e) : rows;
        } else {
            size_t free_b = 0;
            if (xfthip_device_memory(&free_b, nullptr) == 0 && free_b > 0) {
                const double per_value = cfg.kv_dtype == XFTHIP_INT8 ? 1.0 + 4.0 / cfg.head_size : 2.0;
                const double row_b = (double)cfg.layers * 2.0 * cfg.kv_heads * ((maxLen + 1 + 31) / 32 * 32) * cfg.head_size * per_value;
                const double fit_rows_d = 0.4 * (double)free_b / (row_b > 1.0 ? row_b : 1.0);
                rows = fit_rows_d >= 64.0 ? 64 : (fit_rows_d <= 8.0 ? 8 : (int)fit_rows_d);
            }
        }
        const bool grow = model == nullptr || live + add > cfg.max_batch || maxLen + 1 > cfg.max_seq || longestPrompt > cfg.max_tokens;
        if (!grow) return;
        if (live > 0) {
            printf("[ERROR] %d sequences are alive in %d cache rows of %d positions: no room for %d more of length %d.\n", live, cfg.max_batch,
                    cfg.max_seq, add, maxLen);
            exit(-1);
        }
        if (model) CK(xfthip_model_destroy(model)); // rebuilt below with the larger limits
        model = nullptr;
        cfg.max_batch = std::max(std::max(cfg.max_batch, rows), add);
        fit(cfg.max_batch, std::max(longestPrompt, 1), maxLen + 1);
        if (cfg.max_tokens < longestPrompt) {
            printf("[ERROR] internal: token capacity %d below the prompt length %d.\n", cfg.max_tokens, longestPrompt);
            exit(-1);
        }
    }

    ModelImpl() {
        // the reference seeds its sampler from std::random_device on every step (sample_search.cpp:229-231);
        // XFT_SEED makes a run repeatable
        if (const char *e = getenv("XFT_SEED")) rng.seed(strtoull(e, nullptr, 0));
    }

    ~ModelImpl() {
        if (model) xfthip_model_destroy(model);
        drop_moe();
        for (auto &l : L) {
            for (xfthip_weight_t w : {l.qkv, l.o, l.gateup, l.down, l.firstQkv, l.firstO, l.firstGateup, l.firstDown})
                if (w) xfthip_weight_destroy(w);
            for (xfthip_weight_t w : l.expertGateup)
                if (w) xfthip_weight_destroy(w);
            for (xfthip_weight_t w : l.expertDown)
                if (w) xfthip_weight_destroy(w);
        }
        if (lmHead) xfthip_weight_destroy(lmHead);
    }

    // the sparse MLPs work in the first one's buffers: the others go first
    void drop_moe() {
        for (size_t i = moe.size(); i-- > 0;)
            if (moe[i]) xfthip_moe_destroy(moe[i]);
        moe.clear();
    }

    std::string layer_file(int l, const std::string &name) const { return path + "/model.layers." + std::to_string(l) + "." + name; }

    HostMatrix load_matrix(int l, const std::string &stem, int K, int N) const {
        HostMatrix m;
        m.K = K, m.N = N;
        if (fileQuant >= 0) {
            m.qkind = fileQuant;
            m.q = read_bytes(layer_file(l, stem + ".qweight.0.bin"), (size_t)K * N / (fileQuant == XFTHIP_W_UINT4 ? 2 : 1));
            m.zero = read_floats(layer_file(l, stem + ".zeros.0.bin"), N, xft::DataType::fp32);
            m.scale = read_floats(layer_file(l, stem + ".scales.0.bin"), N, xft::DataType::fp32);
        } else {
            m.w = read_floats(layer_file(l, stem + ".weight.0.bin"), (size_t)K * N, fileType);
        }
        return m;
    }

    // Pre-quantised codes go to the device as they are when the requested type is the files' own
    // (MMHelper::convertWeight's INT8->INT8 / UINT4->UINT4 copies, matmul_helper.h:284-315);
    // anything else is dequantised (w = scale * q + zero) and converted like a plain matrix.
    xfthip_weight_t to_device(HostMatrix &m, int flags, int kind = -1) {
        const int wkind = kind >= 0 ? kind : this->wkind;
        xfthip_weight_t h = nullptr;
        if (m.qkind >= 0 && m.qkind == wkind) {
            CK(xfthip_weight_create(wkind, m.K, m.N, m.q.data(), m.scale.data(), m.zero.data(), flags, &h));
        } else {
            if (m.qkind >= 0) {
                m.w.resize((size_t)m.K * m.N);
                for (int k = 0; k < m.K; ++k)
                    for (int n = 0; n < m.N; ++n) {
                        int code;
                        if (m.qkind == XFTHIP_W_UINT4) {
                            const uint8_t b = m.q[((size_t)k * m.N + n) / 2];
                            code = (n & 1) ? (b >> 4) : (b & 15);
                        } else {
                            code = (int8_t)m.q[(size_t)k * m.N + n];
                        }
                        m.w[(size_t)k * m.N + n] = fmaf(m.scale[n], (float)code, m.zero[n]);
                    }
            }
            h = make_weight(wkind, m.K, m.N, m.w.data(), flags);
        }
        weightBytes += xfthip_weight_bytes(h);
        return h;
    }

    void load() {
        const int qCols = heads * headSize, kvCols = kvHeads * headSize, qkvCols = qCols + 2 * kvCols;
        L.resize(layers);
        for (int l = 0; l < layers; ++l) {
            Layer &y = L[l];
            const bool mixed = firstKind >= 0 && firstKind != wkind;
            HostMatrix qkv = load_matrix(l, "attention.query_key_value", hidden, qkvCols);
            y.qkv = to_device(qkv, XFTHIP_WF_NONE);
            if (mixed) y.firstQkv = to_device(qkv, XFTHIP_WF_NONE, firstKind);
            HostMatrix o = load_matrix(l, "attention.dense", qCols, hidden);
            y.o = to_device(o, XFTHIP_WF_NONE);
            if (mixed) y.firstO = to_device(o, XFTHIP_WF_NONE, firstKind);
            if (file_exists(layer_file(l, fileQuant >= 0 ? "mlp.dense_h_to_4h.qweight.0.bin" : "mlp.dense_h_to_4h.weight.0.bin"))) {
                printf("The model directory holds a two-matrix MLP (dense_h_to_4h); only gate/up/down MLPs are served.\n");
                exit(-1);
            }
            if (experts > 0) {
                // loadMixtralFFNWeights (decoder_block.h:640-676): w1 = gate, w2 = up, w3 = down, all [in, out]
                y.router = read_floats(layer_file(l, "moe.gate.weight.bin"), (size_t)hidden * experts, fileType);
                for (int e = 0; e < experts; ++e) {
                    const std::string stem = "moe.sparse_experts." + std::to_string(e) + ".";
                    HostMatrix gate, up, down;
                    gate.K = up.K = hidden, gate.N = up.N = inter, down.K = inter, down.N = hidden;
                    gate.w = read_floats(layer_file(l, stem + "w1.0.bin"), (size_t)hidden * inter, fileType);
                    up.w = read_floats(layer_file(l, stem + "w2.0.bin"), (size_t)hidden * inter, fileType);
                    down.w = read_floats(layer_file(l, stem + "w3.0.bin"), (size_t)inter * hidden, fileType);
                    HostMatrix gu = hcat({&gate, &up});
                    y.expertGateup.push_back(to_device(gu, XFTHIP_WF_GATEUP));
                    y.expertDown.push_back(to_device(down, XFTHIP_WF_NONE));
                }
            } else {
                HostMatrix gate = load_matrix(l, "mlp.gate_proj", hidden, inter);
                HostMatrix up = load_matrix(l, "mlp.up_proj", hidden, inter);
                HostMatrix gu = hcat({&gate, &up});
                // the W8A8 path runs gate/up as one plain GEMM followed by silu(gate) * up
                y.gateup = to_device(gu, wkind == XFTHIP_W_W8A8 ? XFTHIP_WF_NONE : XFTHIP_WF_GATEUP);
                if (mixed) y.firstGateup = to_device(gu, firstKind == XFTHIP_W_W8A8 ? XFTHIP_WF_NONE : XFTHIP_WF_GATEUP, firstKind);
                HostMatrix down = load_matrix(l, "mlp.down_proj", inter, hidden);
                y.down = to_device(down, XFTHIP_WF_NONE);
                if (mixed) y.firstDown = to_device(down, XFTHIP_WF_NONE, firstKind);
            }
            y.ln1 = read_floats(layer_file(l, "input_layernorm.weight.bin"), hidden, fileType);
            y.ln2 = read_floats(layer_file(l, "post_attention_layernorm.weight.bin"), hidden, fileType);
            y.qkvBias = read_floats(layer_file(l, "attention.query_key_value.bias.0.bin"), qkvCols, fileType, false);
            y.oBias = read_floats(layer_file(l, "attention.dense.bias.bin"), hidden, fileType, false);
            if (file_exists(layer_file(l, "mlp.down_proj.bias.0.bin"))) {
                printf("The model directory holds an MLP bias (layer %d); not served.\n", l);
                exit(-1);
            }
        }
        // embedding [vocab, hidden] kept in FP16 (src/layers/token_embedding.h:49-52)
        {
            std::vector<float> e = read_floats(path + "/model.wte.bin", (size_t)vocab * hidden, fileType);
            embedding.resize(e.size());
            for (size_t i = 0; i < e.size(); ++i) embedding[i] = to_fp16(e[i]);
        }
        finalNorm = read_floats(path + "/model.final_layernorm.weight.bin", hidden, fileType);
        // lm_head is stored [vocab, hidden] (trans = true in DistLinear::setWeight, src/layers/dist_linear.h:55-80)
        // and never quantised (common_decoder.h:1000-1001): transposed to [hidden, vocab] bf16 here
        {
            std::vector<float> w = read_floats(path + "/model.lm_head.weight.bin", (size_t)vocab * hidden, fileType);
            std::vector<uint16_t> t((size_t)hidden * vocab);
            for (int v = 0; v < vocab; ++v)
                for (int h = 0; h < hidden; ++h) t[(size_t)h * vocab + v] = to_bf16(w[(size_t)v * hidden + h]);
            CK(xfthip_weight_create(XFTHIP_W_BF16, hidden, vocab, t.data(), nullptr, nullptr, XFTHIP_WF_NONE, &lmHead));
            weightBytes += xfthip_weight_bytes(lmHead);
        }
    }

    // (re)build the device model when a call needs more batch / tokens / positions than it holds
    void fit(int B, int S, int needLen) {
        const bool grow = model == nullptr || B > cfg.max_batch || B * S > cfg.max_tokens || needLen > cfg.max_seq;
        if (!grow) return;
        if (model) CK(xfthip_model_destroy(model));
        model = nullptr;
        prefixOnDevice = false;
        drop_moe();
        cfg.layers = layers, cfg.hidden = hidden, cfg.intermediate = inter;
        cfg.q_heads = heads, cfg.kv_heads = kvHeads, cfg.head_size = headSize;
        cfg.vocab = vocab;
        cfg.max_batch = std::max(cfg.max_batch, B);
        cfg.max_tokens = std::max(cfg.max_tokens, B * S);
        cfg.max_seq = std::max(cfg.max_seq, needLen);
        cfg.max_pos_embed = std::max(maxPosEmbed, cfg.max_seq);
        cfg.rope_base = (int)ropeTheta;
        cfg.kv_dtype = kvDtype;
        cfg.rms_eps = eps;
        CK(xfthip_model_create(&cfg, &model));
        for (int l = 0; l < layers; ++l) {
            Layer &y = L[l];
            if (experts > 0) {
                // MixtralLLM's layer: the attention half and a sparse MLP that carries the post-attention norm weight
                CK(xfthip_model_set_attention(model, l, y.qkv, y.o, y.ln1.data(), y.qkvBias.empty() ? nullptr : y.qkvBias.data(),
                        y.oBias.empty() ? nullptr : y.oBias.data()));
                xfthip_moe_t sparse = nullptr;
                if (moe.empty())
                    CK(xfthip_moe_create(hidden, inter, experts, cfg.max_tokens, y.router.data(), y.ln2.data(), &sparse));
                else
                    CK(xfthip_moe_create_beside(moe[0], y.router.data(), y.ln2.data(), &sparse));
                moe.push_back(sparse);
                for (int e = 0; e < experts; ++e) CK(xfthip_moe_set_expert(sparse, e, y.expertGateup[e], y.expertDown[e]));
                CK(xfthip_model_set_moe(model, l, sparse));
                continue;
            }
            CK(xfthip_model_set_layer(model, l, y.qkv, y.o, y.gateup, y.down, y.ln1.data(), y.ln2.data(),
                    y.qkvBias.empty() ? nullptr : y.qkvBias.data(), y.oBias.empty() ? nullptr : y.oBias.data()));
            if (y.firstQkv) CK(xfthip_model_set_first_token_weights(model, l, y.firstQkv, y.firstO, y.firstGateup, y.firstDown));
        }
        CK(xfthip_model_set_head(model, embedding.data(), finalNorm.data(), lmHead));
    }

    // The prompt pass of a lockstep input.  With a prefix set, the first prefix.size() tokens of every sequence are
    // taken to be the prefix (as the reference takes them, common_decoder.h:337-350) and only the rest runs.
    void prompt_pass(const std::vector<int32_t> &ids, int B, int S, float *logits) {
        if (prefix.empty()) {
            prefixOnDevice = false;
            CK(xfthip_model_prefill(model, ids.data(), B, S, logits, nullptr));
            return;
        }
        const int n = (int)prefix.size(), rest = S - n;
        if (rest <= 0) {
            printf("[ERROR] The input (%d tokens) must be longer than the shared prefix (%d tokens).\n", S, n);
            exit(-1);
        }
        if (!prefixOnDevice) {
            CK(xfthip_model_set_prefix(model, prefix.data(), n, nullptr));
            prefixOnDevice = true;
        }
        std::vector<int32_t> tail((size_t)B * rest);
        for (int b = 0; b < B; ++b) std::copy(ids.begin() + (size_t)b * S + n, ids.begin() + (size_t)(b + 1) * S, tail.begin() + (size_t)b * rest);
        CK(xfthip_model_prefill_after_prefix(model, tail.data(), B, rest, logits, nullptr));
    }

    // ---- searchers ------------------------------------------------------------------------------
    void fetch_logits() {
        const float *dev = nullptr;
        CK(xfthip_model_logits(model, &dev));
        logitsHost.resize((size_t)batch * vocab);
        CK(xfthip_memcpy_d2h(logitsHost.data(), dev, logitsHost.size() * 4, nullptr));
    }

    // search_utils.cpp:22-75 for one rank: the penalised set of a sequence is its prompt plus
    // every token fed back so far
    void repetition_penalty(float *logits) {
        if (step == 1) {
            const int S = (int)output.size() / batch;
            cachedRepetVec.assign(batch, {});
            for (int b = 0; b < batch; ++b) {
                auto &v = cachedRepetVec[b];
                v.assign(output.begin() + (size_t)b * S, output.begin() + (size_t)(b + 1) * S);
                std::sort(v.begin(), v.end());
                v.erase(std::unique(v.begin(), v.end()), v.end());
            }
        } else {
            for (int b = 0; b < batch; ++b) {
                auto &v = cachedRepetVec[b];
                auto it = std::lower_bound(v.begin(), v.end(), nextTokens[b]);
                if (it == v.end() || *it != nextTokens[b]) v.insert(it, nextTokens[b]);
            }
        }
        for (int b = 0; b < batch; ++b)
            for (int idx : cachedRepetVec[b]) {
                if (idx < 0 || idx >= vocab) continue;
                float &x = logits[(size_t)b * vocab + idx];
                x = x < 0 ? x * repetitionPenalty : x / repetitionPenalty;
            }
    }

    // greedy_search.cpp:270-287 / sample_search.cpp:245-265
    void finish_tokens(std::vector<int> &ids) {
        if (eosTokenId != -1)
            for (int b = 0; b < batch; ++b) {
                if (doneBatch[b] == 0) {
                    if (ids[b] == eosTokenId) doneBatch[b] = 1;
                } else if (doneBatch[b] > 0) {
                    ids[b] = padTokenId;
                } else {
                    ids[b] = eosTokenId;
                    doneBatch[b] = 1;
                }
            }
        if (!stopWordsList.empty() && !stopWordsIndex.empty()) {
            // search_utils.cpp:77-99
            for (int b = 0; b < batch; ++b) {
                if (doneBatch[b] != 0) continue;
                for (size_t i = 0; i < stopWordsList.size(); ++i) {
                    auto &words = stopWordsList[i];
                    int &idx = stopWordsIndex[i][b];
                    if (idx < (int)words.size()) {
                        if (words[idx] == ids[b]) {
                            if (++idx == (int)words.size()) doneBatch[b] = -1;
                        } else {
                            idx = 0;
                        }
                    } else {
                        doneBatch[b] = -1;
                    }
                }
            }
        }
    }
};

} // namespace xft

// ---- the deterministic half of SampleSearch::sample (sample_search.cpp:154-226), exported so that it can
// be checked on its own: the top-K candidates of one row (ordered by (value, id) descending, which
// is what partial_sort with greater<pair<float,int>> produces), temperature, the top-P cut with
// the reference's rule (at least 2 candidates; the candidate that crosses topP is left out once more
// than 2 precede it) and the softmax over what is left.  Returns the number of candidates kept.
extern "C" int xft_sample_candidates(const float *logits, int vocab, int topK, float topP, float temperature, int *ids_out,
        float *probs_out) {
    if (topK < 2) topK = 2;
    if (topK > vocab) topK = vocab;
    std::vector<std::pair<float, int>> el(vocab);
    for (int j = 0; j < vocab; ++j) el[j] = std::make_pair(logits[j], j);
    std::partial_sort(el.begin(), el.begin() + topK, el.end(), std::greater<std::pair<float, int>>());
    const float tinv = 1 / temperature;
    std::vector<float> vals(topK);
    for (int j = 0; j < topK; ++j) {
        vals[j] = el[j].first;
        if (tinv != 1.0f) vals[j] *= tinv;
        ids_out[j] = el[j].second;
    }
    int n = topK;
    if (topP < 1.0f) {
        std::vector<float> probs(topK);
        float sum = 0, cur = 0;
        for (int i = 0; i < topK; ++i) {
            probs[i] = expf(vals[i]);
            sum += probs[i];
        }
        const float inv = 1 / sum;
        for (int i = 0; i < topK; ++i) {
            cur += probs[i] * inv;
            if (cur > topP) {
                n = i > 2 ? i : 2;
                break;
            }
        }
    }
    // softmax over the first n values (DecoderUtil::computeSoftmax, src/utils/decoder_util.h:298-340)
    float mx = vals[0];
    for (int i = 1; i < n; ++i) mx = std::max(mx, vals[i]);
    float sum = 0;
    for (int i = 0; i < n; ++i) {
        probs_out[i] = expf(vals[i] - mx);
        sum += probs_out[i];
    }
    const float inv = 1.0f / sum;
    for (int i = 0; i < n; ++i) probs_out[i] *= inv;
    return n;
}

// inverse-CDF draw of sample_search.cpp:232-243: the first candidate whose running sum reaches u
extern "C" int xft_sample_pick(const int *ids, const float *probs, int n, float u) {
    float cur = 0;
    for (int i = 0; i < n; ++i) {
        cur += probs[i];
        if (cur >= u) return ids[i];
    }
    return ids[n - 1]; // rounding left the sum a hair under u
}

namespace xft {

static void unsupported(const char *what) {
    printf("%s is not supported by this build.\n", what);
    exit(-1);
}

Model::Model() : impl(nullptr), batchSize(0), seqLen(0), vocabSize(0), maxSeqLen(0), isNewInput(false) {}

Model::~Model() {
    delete impl;
}

void Model::input(std::vector<int32_t> &inputIds_, int batchSize_) {
    if (impl->cbMode && !impl->pool.empty()) {
        printf("Model::input: %zu sequences of the sequence-id interface are still alive; free them first.\n", impl->pool.size());
        exit(-1);
    }
    impl->cbMode = false;
    if (batchSize_ <= 0 || inputIds_.empty() || inputIds_.size() % (size_t)batchSize_ != 0) {
        printf("Model::input: %zu ids do not form %d sequences of equal length.\n", inputIds_.size(), batchSize_);
        exit(-1);
    }
    isNewInput = true;
    batchSize = batchSize_;
    seqLen = (int)(inputIds_.size() / (size_t)batchSize_);
    inputIds = inputIds_;
}

void Model::config(int maxLen_, int numBeams_, int numBeamHypsToKeep_, float lenPenalty_, bool doEarlyStopping_, int eosTokenId_,
        int padTokenId_, bool doSample_, float temperature_, int topK_, float topP_, float repetitionPenalty_,
        const std::vector<std::vector<int>> &stopWordsList_) {
    configuration.maxLen = maxLen_;
    configuration.numBeams = numBeams_;
    configuration.numBeamHypsToKeep = numBeamHypsToKeep_;
    configuration.lenPenalty = lenPenalty_;
    configuration.doEarlyStopping = doEarlyStopping_;
    configuration.eosTokenId = eosTokenId_;
    configuration.padTokenId = padTokenId_;
    configuration.doSample = doSample_;
    configuration.temperature = temperature_;
    configuration.topK = topK_;
    configuration.topP = topP_;
    configuration.repetitionPenalty = repetitionPenalty_;
    this->config(configuration, stopWordsList_);
}

void Model::config(SearcherConfig &config_, const std::vector<std::vector<int>> &stopWordsList_) {
    isNewInput = true;
    configuration = config_;
    ModelImpl &s = *impl;
    // getGenerationMode: one beam = greedy or sampling, more = beam search (searcher.h)
    if (config_.numBeams < 1) {
        printf("numBeams has to be an integer greater than 0\n");
        exit(-1);
    }
    s.beam = config_.numBeams > 1;
    s.numBeams = config_.numBeams;
    s.numBeamHypsToKeep = config_.numBeamHypsToKeep;
    s.lenPenalty = config_.lenPenalty;
    s.doEarlyStopping = config_.doEarlyStopping;
    if (s.beam && config_.repetitionPenalty != 1.0f)
        printf("[Warning] BeamSearch doesn't support repetition penalty now and repetition penalty is %f.\n", config_.repetitionPenalty);
    s.sampling = config_.doSample && !s.beam;
    s.maxLen = config_.maxLen;
    s.eosTokenId = config_.eosTokenId == -1 ? s.endId : config_.eosTokenId;
    s.padTokenId = config_.padTokenId == -1 ? s.eosTokenId : config_.padTokenId;
    s.repetitionPenalty = config_.repetitionPenalty;
    if (s.repetitionPenalty <= 0) {
        printf("`repetitionPenalty` has to be a strictly positive float, but is %f.\n", s.repetitionPenalty);
        exit(-1);
    }
    if (s.sampling) {
        if (config_.temperature <= 0) {
            printf("Temperature should greater than 0.\n");
            exit(-1);
        }
        s.temperatureInv = 1 / config_.temperature;
        s.topK = config_.topK < 2 ? 2 : config_.topK;
        s.topP = config_.topP;
    }
    s.stopWordsList.clear();
    s.stopWordsIndex.clear();
    s.haveSearcher = true;
    setStopWords(stopWordsList_);
}

bool Model::setStopWords(std::vector<std::vector<int>> stopWordsList) {
    ModelImpl &s = *impl;
    if (s.beam) { // beam_search.cpp:334-337
        if (!stopWordsList.empty()) printf("[Warning] BeamSearch is not supporting stop words yet.\n");
        s.stopWordsList.clear();
        return false;
    }
    // a stop word that is only the EOS token is dropped (greedy_search.cpp:140-146)
    s.stopWordsList.clear();
    for (auto &w : stopWordsList)
        if (!(w.size() == 1 && w[0] == s.eosTokenId)) s.stopWordsList.push_back(w);
    return !s.stopWordsList.empty();
}

bool Model::isDone() {
    ModelImpl &s = *impl;
    if (s.cbMode) {
        for (int id : s.working)
            if (!s.pool.at(id).done) return false;
        return true;
    }
    if (!s.haveSearcher || inputIds.empty()) {
        printf("Please set input and config first.\n");
        exit(-1);
    }
    if (isNewInput) return false;
    if (s.beam) return s.beams.is_done();
    if (s.step == 0) return false;
    if (s.curLen >= s.maxLen) return true;
    for (int f : s.doneBatch)
        if (f <= 0) return false;
    return true;
}

// models.cpp:760-830.  After input(): the prompt pass of the whole batch, (logits, 0, vocab) with the logits of
// the last position of every sequence, or of every position when logitsAll.  After set_input(): one pass of
// the working sequences, all prompts or all decodes, (logits, rows, vocab) with one row a sequence, or one a
// prompt token when logitsAll and the sequences are prompts.
std::tuple<float *, int, int> Model::forward(bool logitsAll) {
    ModelImpl &s = *impl;
    if (s.cbMode) {
        if (s.working.empty()) {
            printf("Please input prompt first.\n");
            exit(-1);
        }
        const int n = (int)s.working.size();
        std::vector<ModelImpl::Seq *> seqs;
        for (int id : s.working) seqs.push_back(&s.pool.at(id));
        const bool prompts = seqs[0]->step == 0;
        for (auto *q : seqs)
            if ((q->step == 0) != prompts) {
                printf("[ERROR] The sequences of one step must be all prompts or all decodes.\n");
                exit(-1);
            }
        if (prompts) {
            size_t total = 0;
            for (auto *q : seqs) total += logitsAll ? q->prompt.size() : 1;
            s.logitsHost.resize(total * s.vocab);
            float *out = s.logitsHost.data();
            for (auto *q : seqs) {
                const int S = (int)q->prompt.size();
                CK(xfthip_model_seq_prefill(s.model, q->row, q->prompt.data(), S, logitsAll ? nullptr : out, nullptr));
                if (logitsAll) CK(xfthip_model_prompt_logits(s.model, 0, S, out, nullptr));
                out += (size_t)(logitsAll ? S : 1) * s.vocab;
            }
            return std::make_tuple(s.logitsHost.data(), (int)total, s.vocab);
        }
        std::vector<int> rows(n);
        for (int i = 0; i < n; ++i) rows[i] = seqs[i]->row;
        CK(xfthip_model_seq_decode(s.model, rows.data(), n, nullptr, nullptr));
        s.logitsHost.resize((size_t)n * s.vocab);
        for (int i = 0; i < n; ++i) CK(xfthip_model_seq_logits(s.model, rows[i], s.logitsHost.data() + (size_t)i * s.vocab));
        return std::make_tuple(s.logitsHost.data(), n, s.vocab);
    }
    if (inputIds.empty() || !isNewInput) unsupported("Model::forward without a new input");
    s.batch = batchSize;
    s.fit(batchSize, seqLen, std::max(seqLen + 1, s.maxLen));
    const size_t rows = logitsAll ? (size_t)batchSize * seqLen : (size_t)batchSize;
    s.logitsHost.resize(rows * s.vocab);
    if (logitsAll && !s.prefix.empty()) unsupported("Model::forward(logitsAll = true) with a shared prefix");
    s.prompt_pass(inputIds, batchSize, seqLen, logitsAll ? nullptr : s.logitsHost.data());
    if (logitsAll) CK(xfthip_model_prompt_logits(s.model, 0, (int)rows, s.logitsHost.data(), nullptr));
    return std::make_tuple(s.logitsHost.data(), 0, s.vocab);
}

// models.cpp:847-903: one step of the working sequences, all prompts or all decodes
static std::vector<int32_t> generate_cb(ModelImpl &s) {
    s.prefixOnDevice = false; // sequences are started in any cache row
    if (s.working.empty()) {
        printf("Please set input tokens by model.set_input().\n");
        exit(-1);
    }
    const int n = (int)s.working.size();
    std::vector<ModelImpl::Seq *> seqs;
    for (int id : s.working) seqs.push_back(&s.pool.at(id));
    const bool prompts = seqs[0]->step == 0;
    for (auto *q : seqs)
        if ((q->step == 0) != prompts) {
            printf("[ERROR] The sequences of one step must be all prompts or all decodes.\n");
            exit(-1);
        }
    std::vector<int> ids(n);
    if (prompts) {
        std::vector<int> all(s.cfg.max_batch);
        for (int i = 0; i < n; ++i) {
            CK(xfthip_model_seq_prefill(s.model, seqs[i]->row, seqs[i]->prompt.data(), (int)seqs[i]->prompt.size(), nullptr, nullptr));
            CK(xfthip_model_last_ids(s.model, all.data(), nullptr));
            ids[i] = all[seqs[i]->row];
        }
    } else {
        std::vector<int> rows(n);
        for (int i = 0; i < n; ++i) rows[i] = seqs[i]->row;
        CK(xfthip_model_seq_decode(s.model, rows.data(), n, ids.data(), nullptr));
    }
    // repetition penalty (search_utils.cpp:103-171) then first-maximum arg-max on the host
    std::vector<float> lg;
    for (int i = 0; i < n; ++i) {
        ModelImpl::Seq &q = *seqs[i];
        if (q.cfg.repetitionPenalty == 1.0f) continue;
        auto &v = q.cachedRepetVec;
        if (q.step == 0) {
            v = std::vector<int>(q.prompt.begin(), q.prompt.end());
            std::sort(v.begin(), v.end());
            v.erase(std::unique(v.begin(), v.end()), v.end());
        } else {
            const int last = q.generated.back();
            auto it = std::lower_bound(v.begin(), v.end(), last);
            if (it == v.end() || *it != last) v.insert(it, last);
        }
        lg.resize(s.vocab);
        CK(xfthip_model_seq_logits(s.model, q.row, lg.data()));
        for (int idx : v) {
            if (idx < 0 || idx >= s.vocab) continue;
            lg[idx] = lg[idx] < 0 ? lg[idx] * q.cfg.repetitionPenalty : lg[idx] / q.cfg.repetitionPenalty;
        }
        int best = 0;
        for (int j = 1; j < s.vocab; ++j)
            if (lg[j] > lg[best]) best = j;
        ids[i] = best;
    }
    // stopCheck (sampling.cpp:134-154), then every sequence steps forward with its token
    for (int i = 0; i < n; ++i) {
        ModelImpl::Seq &q = *seqs[i];
        if (q.done) {
            ids[i] = q.cfg.eosTokenId;
        } else if (ids[i] == q.cfg.eosTokenId) {
            q.done = true;
        } else if ((int)(q.prompt.size() + q.generated.size()) + 1 >= q.cfg.maxLen) {
            q.done = true;
        }
        q.generated.push_back(ids[i]);
        q.step++;
        // the row feeds what the searcher settled on
        if (ids[i] >= 0 && ids[i] < s.vocab) CK(xfthip_model_seq_set_next_id(s.model, q.row, ids[i]));
    }
    return std::vector<int32_t>(ids.begin(), ids.end());
}

// BeamSearch::getNextToken (beam_search.cpp:268-324): the prompt runs once per user sequence, in the cache
// row of its first beam; the other beams' rows are filled from it.  Later steps re-map the generated part of
// the cache rows to the beams the scorer kept, feed every row its token and read all rows' logits.
static std::vector<int32_t> generate_beam(ModelImpl &s, const std::vector<int32_t> &inputIds, int batchSize, int seqLen, bool first) {
    s.prefixOnDevice = false; // the beams' prompts run into cache rows of their own
    const int nb = s.numBeams, rows = batchSize * nb;
    std::vector<int> all(rows);
    for (int i = 0; i < rows; ++i) all[i] = i;
    s.logitsHost.resize((size_t)rows * s.vocab);
    if (first) {
        s.batch = batchSize;
        s.fit(rows, seqLen, std::max(seqLen + 1, s.maxLen) + 1);
        for (int r = 0; r < s.cfg.max_batch; ++r) CK(xfthip_model_seq_release(s.model, r));
        s.beams.start(inputIds.data(), batchSize, seqLen, nb, s.numBeamHypsToKeep, s.maxLen, s.lenPenalty, s.doEarlyStopping, s.eosTokenId,
                s.padTokenId, s.vocab);
        std::vector<int> dst, src;
        for (int b = 0; b < batchSize; ++b) {
            float *lg = s.logitsHost.data() + (size_t)b * nb * s.vocab;
            CK(xfthip_model_seq_prefill(s.model, b * nb, inputIds.data() + (size_t)b * seqLen, seqLen, lg, nullptr));
            for (int j = 1; j < nb; ++j) {
                std::copy(lg, lg + s.vocab, lg + (size_t)j * s.vocab);
                dst.push_back(b * nb + j);
                src.push_back(b * nb);
            }
        }
        CK(xfthip_model_seq_reorder(s.model, dst.data(), src.data(), (int)dst.size(), 0, seqLen, nullptr));
    } else {
        const int cached = s.beams.len - 1; // tokens in every cache row: all but the one about to be fed
        CK(xfthip_model_seq_reorder(s.model, all.data(), s.beams.beamIndices.data(), rows, seqLen, cached, nullptr));
        for (int i = 0; i < rows; ++i) CK(xfthip_model_seq_set_next_id(s.model, i, s.beams.beamTokens[i]));
        CK(xfthip_model_seq_decode(s.model, all.data(), rows, nullptr, nullptr));
        const float *dev = nullptr;
        CK(xfthip_model_logits(s.model, &dev));
        CK(xfthip_memcpy_d2h(s.logitsHost.data(), dev, s.logitsHost.size() * 4, nullptr));
    }
    s.beams.step(s.logitsHost.data());
    s.step++;
    s.curLen = s.beams.len;
    return std::vector<int32_t>(s.beams.beamTokens.begin(), s.beams.beamTokens.end());
}

std::vector<int32_t> Model::generate() {
    ModelImpl &s = *impl;
    if (s.cbMode) return generate_cb(s);
    if (s.beam) {
        if (!s.haveSearcher || inputIds.empty()) {
            printf("Please set input and config first.\n");
            exit(-1);
        }
        const bool first = isNewInput;
        isNewInput = false;
        if (first) s.step = 0;
        return generate_beam(s, inputIds, batchSize, seqLen, first);
    }
    if (!s.haveSearcher) {
        printf("Please set the generation config by model.config().\n");
        exit(-1);
    }
    if (inputIds.empty()) {
        printf("Please set input tokens by model.input().\n");
        exit(-1);
    }
    // the search runs on the host whenever the token is not simply the arg-max of the raw logits
    const bool hostSearch = s.sampling || s.repetitionPenalty != 1.0f;
    if (isNewInput) {
        isNewInput = false;
        s.step = 0;
        s.batch = batchSize;
        s.curLen = seqLen;
        s.doneBatch.assign(batchSize, 0);
        if (!s.stopWordsList.empty()) s.stopWordsIndex.assign(s.stopWordsList.size(), std::vector<int>(batchSize, 0));
        s.output.assign(inputIds.begin(), inputIds.end());
        if (s.maxLen > 0 && seqLen >= s.maxLen) {
            // nothing to generate: the reference still runs the prompt and emits one token
        }
        s.fit(batchSize, seqLen, std::max(seqLen + 1, s.maxLen));
        s.prompt_pass(inputIds, batchSize, seqLen, nullptr);
    } else {
        // feed back what the searcher chose where it differs from the device's own arg-max
        if (s.nextTokens != s.deviceIds) CK(xfthip_model_set_next_ids(s.model, s.nextTokens.data(), nullptr));
        CK(xfthip_model_decode(s.model, 1, nullptr, nullptr));
    }
    s.step++;
    s.deviceIds.resize(batchSize);
    CK(xfthip_model_last_ids(s.model, s.deviceIds.data(), nullptr));
    std::vector<int> ids(batchSize);
    if (!hostSearch) {
        ids = s.deviceIds;
    } else {
        s.fetch_logits();
        if (s.repetitionPenalty != 1.0f) s.repetition_penalty(s.logitsHost.data());
        if (!s.sampling) {
            // first maximum wins (greedy_search.cpp:190-215)
            for (int b = 0; b < batchSize; ++b) {
                const float *p = s.logitsHost.data() + (size_t)b * s.vocab;
                int best = 0;
                for (int j = 1; j < s.vocab; ++j)
                    if (p[j] > p[best]) best = j;
                ids[b] = best;
            }
        } else {
            const int k = std::min(s.topK, s.vocab);
            std::vector<int> cand(k);
            std::vector<float> probs(k);
            std::uniform_real_distribution<float> dist(0.0f, 1.0f);
            for (int b = 0; b < batchSize; ++b) {
                const int n = xft_sample_candidates(s.logitsHost.data() + (size_t)b * s.vocab, s.vocab, s.topK, s.topP,
                        1.0f / s.temperatureInv, cand.data(), probs.data());
                ids[b] = xft_sample_pick(cand.data(), probs.data(), n, dist(s.rng));
            }
        }
    }
    s.finish_tokens(ids);
    s.nextTokens = ids;
    s.curLen++;
    for (int b = 0; b < batchSize; ++b) s.output.insert(s.output.begin() + (size_t)(b + 1) * s.curLen - 1, ids[b]);
    return std::vector<int32_t>(ids.begin(), ids.end());
}

std::vector<int32_t> Model::finalize() {
    ModelImpl &s = *impl;
    if (!s.cbMode && s.beam) return s.beams.finalize();
    if (!s.cbMode) return s.output;
    // models.cpp:738-756: prompt + generated tokens of the working sequences, back to back; their cache
    // rows are released
    std::vector<int32_t> result;
    std::vector<int> ids = s.working;
    for (int id : ids) {
        ModelImpl::Seq &q = s.pool.at(id);
        result.insert(result.end(), q.prompt.begin(), q.prompt.end());
        result.insert(result.end(), q.generated.begin(), q.generated.end());
    }
    freeSeqs(ids);
    return result;
}

// models.cpp:930-946: the prefix runs once; the inputs that follow carry it in front (greedy and sampling in lockstep
// mode; the sequence-id and beam-search paths run whole prompts)
void Model::setPrefix(std::vector<int32_t> &prefixIDs_) {
    ModelImpl &s = *impl;
    if (prefixIDs_.empty()) {
        printf("[ERROR] Model::setPrefix needs at least one token.\n");
        exit(-1);
    }
    s.prefix = prefixIDs_;
    s.prefixOnDevice = false; // run before the next prompt pass (the device model may be rebuilt for it)
}
void Model::unsetPrefix() {
    impl->prefix.clear();
    impl->prefixOnDevice = false;
}
bool Model::freeSeqs(std::vector<int> &seqIDs) {
    ModelImpl &s = *impl;
    bool all = true;
    for (int id : seqIDs) {
        auto it = s.pool.find(id);
        if (it == s.pool.end()) {
            all = false;
            continue;
        }
        CK(xfthip_model_seq_release(s.model, it->second.row));
        s.pool.erase(it);
        s.working.erase(std::remove(s.working.begin(), s.working.end(), id), s.working.end());
    }
    return all;
}

// models.cpp:278-349: new sequences (prompts of any lengths), one pool entry and one cache row each
std::vector<int> Model::set_input(std::vector<std::vector<int32_t>> &inputIds_, SearcherConfig &config_,
        const std::vector<std::vector<int>> &stopWordsList_) {
    std::vector<int> none;
    return set_input(inputIds_, none, config_, stopWordsList_);
}

std::vector<int> Model::set_input(std::vector<int32_t> &inputIds_, int batchSize_, SearcherConfig &config_,
        const std::vector<std::vector<int>> &stopWordsList_) {
    if (batchSize_ <= 0 || inputIds_.size() % (size_t)batchSize_ != 0) {
        printf("Model::set_input: %zu ids do not form %d sequences of equal length.\n", inputIds_.size(), batchSize_);
        exit(-1);
    }
    const size_t len = inputIds_.size() / (size_t)batchSize_;
    std::vector<std::vector<int32_t>> rows;
    for (int b = 0; b < batchSize_; ++b) rows.emplace_back(inputIds_.begin() + b * len, inputIds_.begin() + (b + 1) * len);
    std::vector<int> none;
    return set_input(rows, none, config_, stopWordsList_);
}

// models.cpp:351-410: with no ids, the prompts become new sequences; with ids, those live sequences form
// the batch of the next generate() call (their inputs are the tokens they produced last)
std::vector<int> Model::set_input(std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs, SearcherConfig &config_,
        const std::vector<std::vector<int>> &stopWordsList_) {
    ModelImpl &s = *impl;
    if (!stopWordsList_.empty()) printf("Model::set_input: stop words are not checked on this path (as in the reference).\n");
    if (config_.numBeams != 1) unsupported("Beam search (numBeams != 1)");
    if (config_.doSample) unsupported("Sampling with sequence ids (the reference throws here as well)");
    if (config_.repetitionPenalty <= 0) {
        printf("`repetitionPenalty` has to be a strictly positive float, but is %f.\n", config_.repetitionPenalty);
        exit(-1);
    }
    if (config_.eosTokenId == -1) config_.eosTokenId = s.endId;
    if (config_.padTokenId == -1) config_.padTokenId = config_.eosTokenId;
    if (config_.maxLen < 0) config_.maxLen = maxSeqLen;
    config_.maxLen = std::min(config_.maxLen, maxSeqLen);
    configuration = config_;
    batchSize = (int)inputIds_.size();
    s.cbMode = true;
    s.working.clear();
    if (seqIDs.empty()) {
        int maxLen = config_.maxLen, longest = 0;
        for (auto &ids : inputIds_) {
            if (ids.empty()) {
                printf("[ERROR] Empty prompt.\n");
                exit(-1);
            }
            maxLen = std::max(maxLen, (int)ids.size());
            longest = std::max(longest, (int)ids.size());
        }
        s.fit_rows(batchSize, maxLen, longest);
        for (auto &ids : inputIds_) {
            ModelImpl::Seq q;
            q.id = s.nextSeqId++;
            q.prompt = ids;
            q.cfg = config_;
            q.cfg.maxLen = maxLen;
            q.row = s.free_row();
            if (q.row < 0) {
                printf("[ERROR] No free KV cache row.\n");
                exit(-1);
            }
            s.pool[q.id] = q;
            s.working.push_back(q.id);
            seqIDs.push_back(q.id);
        }
    } else {
        if (inputIds_.size() != seqIDs.size()) {
            printf("[ERROR] Input size and seqIDs size mismatch.\n");
            exit(-1);
        }
        for (int id : seqIDs) {
            if (!s.pool.count(id)) {
                printf("[ERROR] Sequence ID %d not found.\n", id);
                exit(-1);
            }
            s.working.push_back(id);
        }
    }
    return seqIDs;
}

static SearcherConfig flat_config(int maxLen_, int numBeams_, int numBeamHypsToKeep_, float lenPenalty_, bool doEarlyStopping_,
        int eosTokenId_, int padTokenId_, bool doSample_, float temperature_, int topK_, float topP_, float repetitionPenalty_) {
    SearcherConfig c;
    c.maxLen = maxLen_;
    c.numBeams = numBeams_;
    c.numBeamHypsToKeep = numBeamHypsToKeep_;
    c.lenPenalty = lenPenalty_;
    c.doEarlyStopping = doEarlyStopping_;
    c.eosTokenId = eosTokenId_;
    c.padTokenId = padTokenId_;
    c.doSample = doSample_;
    c.temperature = temperature_;
    c.topK = topK_;
    c.topP = topP_;
    c.repetitionPenalty = repetitionPenalty_;
    return c;
}

// models.cpp:238-273: the flat-argument forms fill a SearcherConfig and forward
std::vector<int> Model::set_input(std::vector<int32_t> &inputIds_, int batchSize_, int maxLen_, int numBeams_, int numBeamHypsToKeep_,
        float lenPenalty_, bool doEarlyStopping_, int eosTokenId_, int padTokenId_, bool doSample_, float temperature_, int topK_,
        float topP_, float repetitionPenalty_, const std::vector<std::vector<int>> &stopWordsList_) {
    configuration = flat_config(maxLen_, numBeams_, numBeamHypsToKeep_, lenPenalty_, doEarlyStopping_, eosTokenId_, padTokenId_, doSample_,
            temperature_, topK_, topP_, repetitionPenalty_);
    return set_input(inputIds_, batchSize_, configuration, stopWordsList_);
}

std::vector<int> Model::set_input(std::vector<std::vector<int32_t>> &inputIds_, int maxLen_, int numBeams_, int numBeamHypsToKeep_,
        float lenPenalty_, bool doEarlyStopping_, int eosTokenId_, int padTokenId_, bool doSample_, float temperature_, int topK_,
        float topP_, float repetitionPenalty_, const std::vector<std::vector<int>> &stopWordsList_) {
    configuration = flat_config(maxLen_, numBeams_, numBeamHypsToKeep_, lenPenalty_, doEarlyStopping_, eosTokenId_, padTokenId_, doSample_,
            temperature_, topK_, topP_, repetitionPenalty_);
    return set_input(inputIds_, configuration, stopWordsList_);
}

// ---- the forms "only used for model.forward()" (models.cpp:412-683): sequences without a searcher.  With no
// ids the prompts become new sequences, each with room for its own maximum length; with ids, every listed
// sequence steps forward with the token the caller chose for it (SequenceMeta::stepForward,
// src/common/sequence.h:104-113) and forms the batch of the next forward() call.
static std::vector<int> forward_input(ModelImpl &s, int modelMaxLen, const std::vector<std::vector<int32_t>> &prompts,
        const std::vector<int32_t> &tokens, std::vector<int> seqIDs, const std::vector<int> &maxLens) {
    s.cbMode = true;
    s.working.clear();
    if (seqIDs.empty()) {
        const int n = (int)prompts.size();
        int needLen = 0, longest = 0;
        std::vector<int> lens(n);
        for (int i = 0; i < n; ++i) {
            if (prompts[i].empty()) {
                printf("[ERROR] Empty prompt.\n");
                exit(-1);
            }
            const int want = maxLens.empty() ? -1 : maxLens[maxLens.size() == 1 ? 0 : i];
            lens[i] = want < 0 ? modelMaxLen : std::min(want, modelMaxLen);
            lens[i] = std::max(lens[i], (int)prompts[i].size());
            needLen = std::max(needLen, lens[i]);
            longest = std::max(longest, (int)prompts[i].size());
        }
        s.fit_rows(n, needLen, longest);
        for (int i = 0; i < n; ++i) {
            ModelImpl::Seq q;
            q.id = s.nextSeqId++;
            q.prompt = prompts[i];
            q.forwardOnly = true;
            q.cfg.maxLen = lens[i];
            q.row = s.free_row();
            if (q.row < 0) {
                printf("[ERROR] No free KV cache row.\n");
                exit(-1);
            }
            s.pool[q.id] = q;
            s.working.push_back(q.id);
            seqIDs.push_back(q.id);
        }
        return seqIDs;
    }
    if (tokens.size() != seqIDs.size()) {
        printf("[ERROR] Input size and seqIDs size mismatch.\n");
        exit(-1);
    }
    for (size_t i = 0; i < seqIDs.size(); ++i) {
        auto it = s.pool.find(seqIDs[i]);
        if (it == s.pool.end()) {
            printf("[ERROR] Sequence ID %d not found.\n", seqIDs[i]);
            exit(-1);
        }
        ModelImpl::Seq &q = it->second;
        if (tokens[i] < 0 || tokens[i] >= s.vocab) {
            printf("[ERROR] Token %d of sequence %d is outside the vocabulary.\n", tokens[i], seqIDs[i]);
            exit(-1);
        }
        if ((int)(q.prompt.size() + q.generated.size()) + 1 > s.cfg.max_seq) {
            printf("[ERROR] Sequence ID %d is at the end of its KV cache (%d positions).\n", seqIDs[i], s.cfg.max_seq);
            exit(-1);
        }
        q.generated.push_back(tokens[i]);
        q.step++;
        CK(xfthip_model_seq_set_next_id(s.model, q.row, tokens[i]));
        s.working.push_back(q.id);
    }
    return seqIDs;
}

std::vector<int> Model::set_input(std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs, int maxLen) {
    batchSize = (int)inputIds_.size();
    std::vector<int32_t> tokens;
    if (!seqIDs.empty()) {
        if (inputIds_.size() != seqIDs.size()) {
            printf("[ERROR] Input size and seqIDs size mismatch.\n");
            exit(-1);
        }
        for (auto &ids : inputIds_) {
            if (ids.empty()) {
                printf("[ERROR] Empty input for a sequence.\n");
                exit(-1);
            }
            tokens.push_back(ids[0]);
        }
    }
    return forward_input(*impl, maxSeqLen, inputIds_, tokens, seqIDs, {maxLen});
}

std::vector<int> Model::set_input(std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs, int maxLen) {
    return set_input(inputIds_, batchSize_, seqIDs, std::vector<int> {maxLen});
}

std::vector<int> Model::set_input(std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs, const std::vector<int> &maxLen) {
    if (batchSize_ <= 0 || inputIds_.size() % (size_t)batchSize_ != 0) {
        printf("Model::set_input: %zu ids do not form %d sequences of equal length.\n", inputIds_.size(), batchSize_);
        exit(-1);
    }
    batchSize = batchSize_;
    seqLen = (int)(inputIds_.size() / (size_t)batchSize_);
    if (!(maxLen.size() == (size_t)batchSize || maxLen.size() == 1 || maxLen.empty())) {
        printf("[ERROR] maxLen size and batch size mismatch.\n");
        exit(-1);
    }
    std::vector<std::vector<int32_t>> prompts;
    if (seqIDs.empty()) {
        for (int b = 0; b < batchSize_; ++b) prompts.emplace_back(inputIds_.begin() + (size_t)b * seqLen, inputIds_.begin() + (size_t)(b + 1) * seqLen);
    } else if (inputIds_.size() != (size_t)batchSize_) {
        printf("[ERROR] Input size and batch size mismatch.\n");
        exit(-1);
    }
    return forward_input(*impl, maxSeqLen, prompts, inputIds_, seqIDs, maxLen);
}

std::vector<int> Model::set_input(std::vector<int32_t> &inputIds_, std::vector<int32_t> &seqLens_, std::vector<int> seqIDs,
        std::vector<int> &maxLen) {
    std::vector<std::vector<int32_t>> prompts;
    if (seqIDs.empty()) {
        batchSize = (int)seqLens_.size();
        if (!(maxLen.size() == (size_t)batchSize || maxLen.size() == 1 || maxLen.empty())) {
            printf("[ERROR] maxLen size and batch size mismatch.\n");
            exit(-1);
        }
        size_t at = 0;
        for (int len : seqLens_) {
            if (len < 0 || at + (size_t)len > inputIds_.size()) {
                printf("[ERROR] seqLens do not fit the %zu input ids.\n", inputIds_.size());
                exit(-1);
            }
            prompts.emplace_back(inputIds_.begin() + at, inputIds_.begin() + at + len);
            at += (size_t)len;
        }
    } else {
        batchSize = (int)seqIDs.size();
    }
    return forward_input(*impl, maxSeqLen, prompts, inputIds_, seqIDs, maxLen);
}

// models.cpp:905-935: the searcher half of config(), without the stop words
void Model::createSearcher(SearcherConfig &config_) {
    this->config(config_, {});
}

void Model::initMaxSeqLen() {
    maxSeqLen = impl->maxSeqLength > 0 ? impl->maxSeqLength : impl->maxPositions;
}

AutoModel::AutoModel(std::string modelPath, xft::DataType dataType, xft::DataType KVCacheDataType) : Model() {
    const std::string configPath = modelPath + "/config.ini";
    Ini ini(configPath);
    if (!ini.ok || ini.sections.empty()) {
        printf("Could not load model config.ini.\n");
        exit(-1);
    }
    const std::string sec = *ini.sections.begin();
    setVocabSize((int)ini.get_int(sec, "vocab_size", 0));

    const std::string modelKey = sec + "-" + type_name(dataType) + "-" + type_name(KVCacheDataType);
    // one weight type, or FirstTokenDtype_NextTokenDtype (HybridModel, models.cpp:1014-1035 with the
    // registry keys of src/models/*.cpp)
    int wkind = -1, firstKind = -1;
    switch (dataType) {
        case xft::DataType::bf16:
        case xft::DataType::fp16:
        case xft::DataType::int8:
        case xft::DataType::w8a8:
        case xft::DataType::int4:
        case xft::DataType::nf4: wkind = kind_of(dataType); break;
        case xft::DataType::bf16_fp16: firstKind = kind_of(xft::DataType::bf16), wkind = kind_of(xft::DataType::fp16); break;
        case xft::DataType::bf16_int8: firstKind = kind_of(xft::DataType::bf16), wkind = kind_of(xft::DataType::int8); break;
        case xft::DataType::bf16_w8a8: firstKind = kind_of(xft::DataType::bf16), wkind = kind_of(xft::DataType::w8a8); break;
        case xft::DataType::bf16_int4: firstKind = kind_of(xft::DataType::bf16), wkind = kind_of(xft::DataType::int4); break;
        case xft::DataType::bf16_nf4: firstKind = kind_of(xft::DataType::bf16), wkind = kind_of(xft::DataType::nf4); break;
        case xft::DataType::w8a8_int8: firstKind = kind_of(xft::DataType::w8a8), wkind = kind_of(xft::DataType::int8); break;
        case xft::DataType::w8a8_int4: firstKind = kind_of(xft::DataType::w8a8), wkind = kind_of(xft::DataType::int4); break;
        case xft::DataType::w8a8_nf4: firstKind = kind_of(xft::DataType::w8a8), wkind = kind_of(xft::DataType::nf4); break;
        default: break; // fp8_e4m3 and unknown
    }
    const bool kvOk = KVCacheDataType == xft::DataType::fp16 || KVCacheDataType == xft::DataType::int8;
    const bool mixtral = Ini::lower(sec) == "mixtral";
    if ((Ini::lower(sec) != "llama" && !mixtral) || wkind < 0 || !kvOk) {
        printf("Unsupported data type or KV cache data type: %s\n", modelKey.c_str());
        exit(-1);
    }
    if (mixtral && (firstKind >= 0 || wkind == XFTHIP_W_W8A8)) {
        // (the experts run the weight-only GEMMs with the fused SwiGLU; one weight set)
        printf("Unsupported data type for a sparse-MLP model: %s\n", modelKey.c_str());
        exit(-1);
    }

    ensure_init();
    impl = new ModelImpl();
    ModelImpl &s = *impl;
    s.path = modelPath;
    s.modelType = sec;
    s.wkind = wkind;
    s.firstKind = firstKind;
    s.kvDtype = KVCacheDataType == xft::DataType::int8 ? XFTHIP_INT8 : XFTHIP_FP16;
    // the keys and defaults of CommonDecoder's constructor (common_decoder.h:176-212)
    s.heads = (int)ini.get_int(sec, "head_num", 0);
    s.kvHeads = (int)ini.get_int(sec, "kv_head_num", s.heads);
    s.headSize = (int)ini.get_int(sec, "size_per_head", 0);
    s.inter = (int)ini.get_int(sec, "inter_size", 0);
    s.layers = (int)ini.get_int(sec, "num_layer", 0);
    s.vocab = (int)ini.get_int(sec, "vocab_size", 0);
    s.maxPosEmbed = (int)ini.get_int(sec, "max_pos_seq_len", 0);
    s.maxPositions = (int)ini.get_int(sec, "model_max_length", s.maxPosEmbed);
    s.maxSeqLength = (int)ini.get_int(sec, "seq_length", -1);
    s.hidden = (int)ini.get_int(sec, "hidden_size", (long)s.heads * s.headSize);
    s.eps = (float)ini.get_float(sec, "layernorm_eps", 1e-6);
    s.ropeTheta = (float)ini.get_float(sec, "rope_theta", 10000.0);
    s.experts = mixtral ? (int)ini.get_int(sec, "sparse_experts", 8) : 0; // common_decoder.h:249
    s.startId = (int)ini.get_int(sec, "start_id", 0);
    s.endId = (int)ini.get_int(sec, "end_id", s.startId);
    if (s.heads <= 0 || s.headSize <= 0 || s.inter <= 0 || s.layers <= 0 || s.vocab <= 0 || s.hidden <= 0) {
        printf("config.ini of %s lacks head_num / size_per_head / inter_size / num_layer / vocab_size.\n", modelPath.c_str());
        exit(-1);
    }
    const std::string ropeType = ini.get(sec, "rope_scaling_type", "");
    if (!ropeType.empty() && Ini::lower(ropeType) != "null" && Ini::lower(ropeType) != "none") {
        printf("rope_scaling_type = %s is not supported by this build.\n", ropeType.c_str());
        exit(-1);
    }
    std::string act = Ini::lower(ini.get(sec, "activation_type", "silu"));
    if (act != "silu" && act != "swiglu") {
        printf("activation_type = %s is not supported by this build.\n", act.c_str());
        exit(-1);
    }
    // element type of the plain files (weight_util.h:37-67)
    const std::string wt = ini.get(sec, "weight_data_type", "fp32");
    if (wt.find("fp32") != std::string::npos) s.fileType = xft::DataType::fp32;
    else if (wt.find("fp16") != std::string::npos) s.fileType = xft::DataType::fp16;
    else if (wt.find("bf16") != std::string::npos) s.fileType = xft::DataType::bf16;
    else {
        printf("Invalid type %s. Use FP32 as default", wt.c_str());
        s.fileType = xft::DataType::fp32;
    }
    // pre-quantised directories (common_decoder.h:214-233)
    const std::string qt = ini.get(sec, "quant_qweight_data_type", "");
    if (qt == "int8" || qt == "uint4") {
        s.fileQuant = qt == "int8" ? XFTHIP_W_INT8 : XFTHIP_W_UINT4;
        if (ini.get(sec, "quant_scales_data_type", "") != "fp32") {
            printf("scales should be fp32 data type.\n");
            exit(-1);
        }
        if (ini.get(sec, "quant_zeros_data_type", "") != "fp32") {
            printf("zeros should be fp32 data type.\n");
            exit(-1);
        }
        if (ini.get_int(sec, "quant_groupsize", -1) != -1) {
            printf("Quantization with groupsize is not supported.\n");
            exit(-1);
        }
        if (mixtral) {
            printf("Pre-quantised sparse-MLP model directories are not supported by this build.\n");
            exit(-1);
        }
    }
    s.load();
    maxSeqLen = s.maxSeqLength > 0 ? s.maxSeqLength : s.maxPositions;
}

} // namespace xft

// ---- C entry points for language bindings (the role of the reference's Torch custom class,
// src/pytorch/auto_model.h): one opaque handle per AutoModel ----------------------------------------
extern "C" {

static xft::DataType dtype_from_name(const char *name) {
    static const char *names[] = {"fp32", "bf16", "fp16", "int8", "w8a8", "int4", "nf4", "bf16_fp16", "bf16_int8", "bf16_w8a8",
            "bf16_int4", "bf16_nf4", "w8a8_int8", "w8a8_int4", "w8a8_nf4", "fp8_e4m3"};
    for (int i = 0; i < 16; ++i)
        if (strcmp(name, names[i]) == 0) return (xft::DataType)i;
    return xft::DataType::unknown;
}

void *xft_automodel_create(const char *path, const char *dtype, const char *kv_dtype) {
    return new xft::AutoModel(path, dtype_from_name(dtype), dtype_from_name(kv_dtype));
}

void xft_automodel_destroy(void *h) {
    delete (xft::AutoModel *)h;
}

// stop words arrive flattened: n_words lengths, then the ids back to back
void xft_automodel_config(void *h, int maxLen, int numBeams, int numBeamHypsToKeep, float lenPenalty, int doEarlyStopping,
        int eosTokenId, int padTokenId, int doSample, float temperature, int topK, float topP, float repetitionPenalty,
        const int *stop_lens, const int *stop_ids, int n_words) {
    std::vector<std::vector<int>> words;
    int off = 0;
    for (int i = 0; i < n_words; ++i) {
        words.emplace_back(stop_ids + off, stop_ids + off + stop_lens[i]);
        off += stop_lens[i];
    }
    ((xft::AutoModel *)h)->config(maxLen, numBeams, numBeamHypsToKeep, lenPenalty, doEarlyStopping != 0, eosTokenId, padTokenId,
            doSample != 0, temperature, topK, topP, repetitionPenalty, words);
}

void xft_automodel_input(void *h, const int *ids, int batch, int seq_len) {
    std::vector<int32_t> v(ids, ids + (size_t)batch * seq_len);
    ((xft::AutoModel *)h)->input(v, batch);
}

// one generation step; next_out holds batch ids
int xft_automodel_generate(void *h, int *next_out) {
    std::vector<int32_t> r = ((xft::AutoModel *)h)->generate();
    memcpy(next_out, r.data(), r.size() * 4);
    return (int)r.size();
}

int xft_automodel_is_done(void *h) {
    return ((xft::AutoModel *)h)->isDone() ? 1 : 0;
}

// Two-call protocol: out = NULL finalizes (which also frees continuously batched sequences) and returns
// the number of ids; the next call with a buffer copies them out.
int xft_automodel_finalize(void *h, int *out, int capacity) {
    static std::map<void *, std::vector<int32_t>> pending;
    if (out == nullptr || !pending.count(h)) pending[h] = ((xft::AutoModel *)h)->finalize();
    std::vector<int32_t> &r = pending[h];
    const int n = (int)r.size();
    if (out) {
        memcpy(out, r.data(), (size_t)std::min(n, capacity) * 4);
        pending.erase(h);
    }
    return n;
}

// logits of the prompt's next token, fp32 [batch, vocab] (Model::forward(false))
int xft_automodel_forward(void *h, float *logits_out) {
    auto t = ((xft::AutoModel *)h)->forward(false);
    xft::AutoModel *m = (xft::AutoModel *)h;
    memcpy(logits_out, std::get<0>(t), (size_t)m->getBatchSize() * std::get<2>(t) * 4);
    return std::get<2>(t);
}

// Continuous batching.  Prompts arrive flattened (n lengths, then the ids back to back); seq_ids may be
// NULL (n_ids = 0: new sequences).  Returns the number of sequence ids written to ids_out.
int xft_automodel_set_input(void *h, const int *lens, const int *ids, int n, const int *seq_ids, int n_ids, int maxLen, int eosTokenId,
        int padTokenId, float repetitionPenalty, int *ids_out) {
    std::vector<std::vector<int32_t>> prompts;
    int off = 0;
    for (int i = 0; i < n; ++i) {
        prompts.emplace_back(ids + off, ids + off + lens[i]);
        off += lens[i];
    }
    SearcherConfig cfg(maxLen, 1, 1, 1.0f, false, eosTokenId, padTokenId, false, 1.0f, 50, 1.0f, repetitionPenalty);
    std::vector<int> given(seq_ids, seq_ids + n_ids);
    std::vector<int> out = ((xft::AutoModel *)h)->set_input(prompts, given, cfg, {});
    memcpy(ids_out, out.data(), out.size() * 4);
    return (int)out.size();
}

// n > 0: Model::setPrefix with these ids; n == 0: Model::unsetPrefix
void xft_automodel_set_prefix(void *h, const int *ids, int n) {
    if (n <= 0) {
        ((xft::AutoModel *)h)->unsetPrefix();
        return;
    }
    std::vector<int32_t> v(ids, ids + n);
    ((xft::AutoModel *)h)->setPrefix(v);
}

int xft_automodel_free_seqs(void *h, const int *seq_ids, int n) {
    std::vector<int> v(seq_ids, seq_ids + n);
    return ((xft::AutoModel *)h)->freeSeqs(v) ? 1 : 0;
}

// The beam searcher's host half on its own (no device): a test feeds it logits and reads its choices.
void *xft_beam_create(const int *prompt_ids, int batch, int seq_len, int num_beams, int keep, int max_len, float len_penalty, int early,
        int eos, int pad, int vocab) {
    xft::BeamSearcher *b = new xft::BeamSearcher();
    b->start(prompt_ids, batch, seq_len, num_beams, keep, max_len, len_penalty, early != 0, eos, pad, vocab);
    return b;
}
// logits fp32 [batch * num_beams, vocab] (overwritten); tokens_out / indices_out int32 [batch * num_beams]
void xft_beam_step(void *h, float *logits, int *tokens_out, int *indices_out, float *scores_out) {
    xft::BeamSearcher *b = (xft::BeamSearcher *)h;
    b->step(logits);
    memcpy(tokens_out, b->beamTokens.data(), b->beamTokens.size() * 4);
    memcpy(indices_out, b->beamIndices.data(), b->beamIndices.size() * 4);
    if (scores_out) memcpy(scores_out, b->beamScores.data(), b->beamScores.size() * 4);
}
int xft_beam_is_done(void *h) {
    return ((xft::BeamSearcher *)h)->is_done() ? 1 : 0;
}
// returns the number of ids (batch * keep * row length); copies at most `capacity`; call once
int xft_beam_finalize(void *h, int *out, int capacity) {
    std::vector<int32_t> r = ((xft::BeamSearcher *)h)->finalize();
    memcpy(out, r.data(), (size_t)std::min((int)r.size(), capacity) * 4);
    return (int)r.size();
}
void xft_beam_destroy(void *h) {
    delete (xft::BeamSearcher *)h;
}

int xft_automodel_vocab_size(void *h) {
    return ((xft::AutoModel *)h)->getVocabSize();
}

int xft_automodel_max_seq_len(void *h) {
    return ((xft::AutoModel *)h)->getMaxSeqLen();
}

} // extern "C"
