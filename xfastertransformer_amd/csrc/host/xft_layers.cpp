// Host side of the drop-in boundary: the reference's public layer entry points
// (include/layers_*.h, namespace xft) implemented over the C-ABI of the gfx950 library.
// Plain C++ (g++), no HIP headers: everything device-side goes through include/xft_hip.h.
//
// Conventions kept from the reference (src/layers/decoder_layer.cpp, attention.cpp,
// mlp_llama.cpp): void functions that print and exit(-1) on failure; a function-local static
// mutex serialises each invoke*LLaMA; weights are fp32 host matrices [in, out], converted once
// on first sight and cached for the life of the process under a key made of their addresses
// plus dims and dt; activations are fp32 host buffers; the KV cache (FP16) is owned here and
// the caller supplies pastSeqLen / step.  Beyond the reference: dt may also be int8, w8a8, int4
// or nf4, which selects the weight-only / W8A8 formats (the reference's entry points print
// ">> unsupported data type" for every dt but bf16 / fp16, decoder_layer.cpp:172-206).
// dt = fp16 is served with the weights narrowed to bf16 (8 significant bits instead of fp16's
// 11): this build has no fp16 weight kind; a one-line notice says so once.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../../include/layers_attention.h"
#include "../../../include/layers_decoder.h"
#include "../../../include/layers_gemm.h"
#include "../../../include/layers_mlp.h"
#include "../../../include/layers_norm.h"
#include "../../../include/layers_rotary_embedding.h"
#include "../../../include/xft_hip.h"
#include "host_util.h"

using namespace xfthost;

namespace {

// Gather Q | K | V column blocks (row stride = qkvCols, src/layers/attention.h:122-136) into one
// contiguous [hidden, qkvCols] matrix.
std::vector<float> concat_qkv(const float *q, const float *k, const float *v, int hidden, int qCols, int kvCols) {
    const int stride = qCols + 2 * kvCols;
    std::vector<float> out((size_t)hidden * stride);
    for (int i = 0; i < hidden; ++i) {
        memcpy(&out[(size_t)i * stride], q + (size_t)i * stride, sizeof(float) * qCols);
        memcpy(&out[(size_t)i * stride + qCols], k + (size_t)i * stride, sizeof(float) * kvCols);
        memcpy(&out[(size_t)i * stride + qCols + kvCols], v + (size_t)i * stride, sizeof(float) * kvCols);
    }
    return out;
}

std::vector<float> concat_bias(const float *q, const float *k, const float *v, int qCols, int kvCols) {
    std::vector<float> out;
    if (!q && !k && !v) return out;
    out.assign((size_t)qCols + 2 * kvCols, 0.0f);
    if (q) memcpy(out.data(), q, sizeof(float) * qCols);
    if (k) memcpy(out.data() + qCols, k, sizeof(float) * kvCols);
    if (v) memcpy(out.data() + qCols + kvCols, v, sizeof(float) * kvCols);
    return out;
}

// cat(gate, up) as LlamaMLP::catGateUpWeights lays it out: [hidden, 2 * inter]
std::vector<float> concat_gateup(const float *gate, const float *up, int hidden, int inter) {
    std::vector<float> out((size_t)hidden * 2 * inter);
    for (int i = 0; i < hidden; ++i) {
        memcpy(&out[(size_t)i * 2 * inter], gate + (size_t)i * inter, sizeof(float) * inter);
        memcpy(&out[(size_t)i * 2 * inter + inter], up + (size_t)i * inter, sizeof(float) * inter);
    }
    return out;
}

struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    void *get(size_t bytes) {
        if (bytes > cap) {
            if (p) xfthip_free(p);
            CK(xfthip_malloc(&p, bytes));
            cap = bytes;
        }
        return p;
    }
};

// One cached layer: a 1-layer device model plus the weight handles it references.
struct Entry {
    xfthip_model_t model = nullptr;
    xfthip_weight_t qkv = nullptr, o = nullptr, gateup = nullptr, down = nullptr;
    std::vector<float> ln1, ln2, qkvBias, oBias;
    std::vector<float> ln1Beta, ln2Beta; // NormType::LN layers only
    xfthip_model_config cfg {};
    bool hasAttn = false, hasMlp = false;
};

void build_model(Entry &e) {
    if (e.model) CK(xfthip_model_destroy(e.model));
    e.model = nullptr;
    CK(xfthip_model_create(&e.cfg, &e.model));
    if (e.hasAttn)
        CK(xfthip_model_set_attention(e.model, 0, e.qkv, e.o, e.ln1.empty() ? nullptr : e.ln1.data(),
                e.qkvBias.empty() ? nullptr : e.qkvBias.data(), e.oBias.empty() ? nullptr : e.oBias.data()));
    if (e.hasMlp) CK(xfthip_model_set_mlp(e.model, 0, e.gateup, e.down, e.ln2.empty() ? nullptr : e.ln2.data()));
    if (!e.ln1Beta.empty()) CK(xfthip_model_set_layer_norm_shifts(e.model, 0, e.ln1Beta.data(), e.ln2Beta.data()));
}

// grow the model when a call needs more batch / tokens / positions than it was built for
void fit_model(Entry &e, int batch, int tokens, int maxPositions, int maxPosEmbed) {
    bool rebuild = e.model == nullptr;
    if (batch > e.cfg.max_batch) { e.cfg.max_batch = batch; rebuild = true; }
    if (tokens > e.cfg.max_tokens) { e.cfg.max_tokens = tokens; rebuild = true; }
    if (maxPositions > e.cfg.max_seq) { e.cfg.max_seq = maxPositions; rebuild = true; }
    if (maxPosEmbed > e.cfg.max_pos_embed) { e.cfg.max_pos_embed = maxPosEmbed; rebuild = true; }
    if (e.cfg.max_pos_embed < e.cfg.max_seq) { e.cfg.max_pos_embed = e.cfg.max_seq; rebuild = true; }
    if (e.cfg.max_tokens < e.cfg.max_batch) { e.cfg.max_tokens = e.cfg.max_batch; rebuild = true; }
    if (rebuild) build_model(e);
}

// upload fp32 rows, run `body(dev_in, dev_out)` (dense [rows, cols] device buffers), download
void run_rows(const void *input, int inputStride, void *output, int outputStride, int rows, int cols,
        const std::function<void(const float *, float *)> &body) {
    static DevBuf din, dout;
    std::vector<float> dense((size_t)rows * cols);
    for (int r = 0; r < rows; ++r) memcpy(&dense[(size_t)r * cols], (const float *)input + (size_t)r * inputStride, sizeof(float) * cols);
    float *di = (float *)din.get(dense.size() * sizeof(float));
    float *dop = (float *)dout.get(dense.size() * sizeof(float));
    CK(xfthip_memcpy_h2d(di, dense.data(), dense.size() * sizeof(float), nullptr));
    body(di, dop);
    CK(xfthip_memcpy_d2h(dense.data(), dop, dense.size() * sizeof(float), nullptr));
    for (int r = 0; r < rows; ++r) memcpy((float *)output + (size_t)r * outputStride, &dense[(size_t)r * cols], sizeof(float) * cols);
}

} // namespace

namespace xft {

void invokeLayerLLaMA(DataType dt, ActivationType at, NormType nt, int batchSize, int inputSeqLen, int attHeadDim,
        int attHeadNum, int kvHeadNum, int maxPositions, int maxPosEmbed, int pastSeqLen, int currentSeqLen, int step,
        int hiddenSize, int intermediateSize, void *output, int outputStride, const void *input, int inputStride,
        const float *ln1Gamma, const float *ln1Beta, const void *queryWeight, const void *keyWeight,
        const void *valueWeight, const void *attnOutWeight, const float *ln2Gamma, const float *ln2Beta,
        const void *gateWeight, const void *upWeight, const void *downWeight, const float *queryBias,
        const float *keyBias, const float *valueBias, const float *attnOutBias) {
    static std::mutex mutex;
    std::lock_guard<std::mutex> lock(mutex);
    (void)currentSeqLen; (void)step;

    const int kind = kind_of(dt);
    if (kind < 0) return; // message printed, output untouched, as the reference (decoder_layer.cpp:172-206)
    if (nt != NormType::RMS && nt != NormType::LN) {
        printf(">> unsupported norm type\n");
        return;
    }
    if (nt == NormType::LN && (!ln1Beta || !ln2Beta)) {
        printf(">> NormType::LN needs ln1Beta and ln2Beta\n");
        exit(-1);
    }
    if (at != ActivationType::SILU && at != ActivationType::SWIGLU) {
        printf(">> unsupported activation type\n");
        return;
    }
    ensure_init();

    static std::unordered_map<std::string, Entry> hub;
    std::stringstream key;
    key << queryWeight << "_" << keyWeight << "_" << valueWeight << "_" << attnOutWeight << "_" << gateWeight << "_" << upWeight
        << "_" << downWeight << "_" << dt << "_" << at << "_" << nt << "_" << attHeadDim << "_" << attHeadNum << "_" << kvHeadNum;
    Entry &e = hub[key.str()];
    if (!e.hasAttn) {
        const int qCols = attHeadNum * attHeadDim, kvCols = kvHeadNum * attHeadDim;
        auto qkv = concat_qkv((const float *)queryWeight, (const float *)keyWeight, (const float *)valueWeight, hiddenSize, qCols, kvCols);
        e.qkv = make_weight(kind, hiddenSize, qCols + 2 * kvCols, qkv.data(), XFTHIP_WF_NONE);
        e.o = make_weight(kind, qCols, hiddenSize, (const float *)attnOutWeight, XFTHIP_WF_NONE);
        auto gu = concat_gateup((const float *)gateWeight, (const float *)upWeight, hiddenSize, intermediateSize);
        e.gateup = make_weight(kind, hiddenSize, 2 * intermediateSize, gu.data(), kind == XFTHIP_W_W8A8 ? XFTHIP_WF_NONE : XFTHIP_WF_GATEUP);
        e.down = make_weight(kind, intermediateSize, hiddenSize, (const float *)downWeight, XFTHIP_WF_NONE);
        e.ln1.assign(ln1Gamma, ln1Gamma + hiddenSize);
        e.ln2.assign(ln2Gamma, ln2Gamma + hiddenSize);
        if (nt == NormType::LN) {
            // the layer over LayerNorm instead of RmsNorm (decoder_layer.cpp:179-181, 195-197)
            e.ln1Beta.assign(ln1Beta, ln1Beta + hiddenSize);
            e.ln2Beta.assign(ln2Beta, ln2Beta + hiddenSize);
        }
        e.qkvBias = concat_bias(queryBias, keyBias, valueBias, qCols, kvCols);
        if (attnOutBias) e.oBias.assign(attnOutBias, attnOutBias + hiddenSize);
        e.hasAttn = e.hasMlp = true;
        e.cfg = xfthip_model_config {1, hiddenSize, intermediateSize, attHeadNum, kvHeadNum, attHeadDim, 0, batchSize, maxPositions,
                batchSize * inputSeqLen, maxPosEmbed, 10000, XFTHIP_FP16, 1e-6f};
        printf(">> create llama_layer_key: %s\n", key.str().c_str());
    }
    fit_model(e, batchSize, batchSize * inputSeqLen, maxPositions, maxPosEmbed);
    run_rows(input, inputStride, output, outputStride, batchSize * inputSeqLen, hiddenSize, [&](const float *di, float *dop) {
        CK(xfthip_model_layer_forward(e.model, 0, di, hiddenSize, dop, hiddenSize, batchSize, inputSeqLen, pastSeqLen, nullptr));
    });
}

void invokeAttention(DataType dt, void *output, const void *query, const void *key, const void *value, int *query_shape,
        int *kv_shape, const int q_stride, const int kv_stride, const float scale, const int batch_size,
        const int *token_lens, const void *kcache, const void *vcache, int *kvcache_shape, int *block_tables,
        int *block_nums, int *context_lens, int layer_id, bool is_prefill, int *slot_mapping) {
    static std::mutex mutex;
    std::lock_guard<std::mutex> lock(mutex);
    (void)layer_id;
    if (dt != DataType::bf16) {
        printf("Error: data type (%d) is not supported yet!\n", dt);
        exit(-1);
    }
    ensure_init();
    const int total = query_shape[0], qHeads = query_shape[1], headSize = query_shape[2], kvHeads = kv_shape[1];
    const int blockNum = kvcache_shape[0], blockSize = kvcache_shape[1];
    if (kvcache_shape[2] != kvHeads || kvcache_shape[3] != headSize || batch_size <= 0 || total <= 0) {
        printf("invokeAttention: kvcache_shape [%d, %d, %d, %d] does not match %d KV heads of size %d\n", kvcache_shape[0],
                kvcache_shape[1], kvcache_shape[2], kvcache_shape[3], kvHeads, headSize);
        exit(-1);
    }
    const size_t rowElems = (size_t)kvHeads * headSize, cacheBytes = (size_t)blockNum * blockSize * rowElems * 2;
    // device copies of the caches, keyed by the host address
    struct Mirror {
        void *dev = nullptr;
        size_t bytes = 0;
    };
    static std::unordered_map<const void *, Mirror> mirrors;
    auto mirror_of = [&](const void *host) {
        Mirror &m = mirrors[host];
        if (m.bytes != cacheBytes) {
            if (m.dev) xfthip_free(m.dev);
            CK(xfthip_malloc(&m.dev, cacheBytes));
            CK(xfthip_memcpy_h2d(m.dev, host, cacheBytes, nullptr));
            m.bytes = cacheBytes;
        }
        return m.dev;
    };
    void *kc = mirror_of(kcache), *vc = mirror_of(vcache);

    const int oStride = qHeads * headSize;
    int rows = total;
    if (!is_prefill) rows = batch_size;
    static DevBuf dq, dk, dv, dout, dtab, dctx, dslot;
    CK(xfthip_memcpy_h2d(dq.get((size_t)rows * q_stride * 2), query, ((size_t)(rows - 1) * q_stride + (size_t)qHeads * headSize) * 2, nullptr));
    CK(xfthip_memcpy_h2d(dk.get((size_t)rows * kv_stride * 2), key, ((size_t)(rows - 1) * kv_stride + rowElems) * 2, nullptr));
    CK(xfthip_memcpy_h2d(dv.get((size_t)rows * kv_stride * 2), value, ((size_t)(rows - 1) * kv_stride + rowElems) * 2, nullptr));
    CK(xfthip_memcpy_h2d(dslot.get((size_t)rows * 4), slot_mapping, (size_t)rows * 4, nullptr));
    dout.get((size_t)rows * oStride * 2);
    if (!is_prefill) {
        int maxCtx = 0, tableStride = 0;
        for (int b = 0; b < batch_size; ++b) {
            if (context_lens[b] > maxCtx) maxCtx = context_lens[b];
            const int nb = block_nums ? block_nums[b] : context_lens[b] / blockSize + 1;
            if (nb > tableStride) tableStride = nb;
            if (nb * blockSize < context_lens[b] + 1) {
                printf("invokeAttention: sequence %d has %d blocks of %d for %d + 1 tokens\n", b, nb, blockSize, context_lens[b]);
                exit(-1);
            }
        }
        CK(xfthip_memcpy_h2d(dtab.get((size_t)batch_size * tableStride * 4), block_tables, (size_t)batch_size * tableStride * 4, nullptr));
        CK(xfthip_memcpy_h2d(dctx.get((size_t)batch_size * 4), context_lens, (size_t)batch_size * 4, nullptr));
        CK(xfthip_paged_attention_decode(dout.p, dq.p, dk.p, dv.p, qHeads, kvHeads, headSize, q_stride, kv_stride, oStride, scale, batch_size,
                kc, vc, blockNum, blockSize, (const int *)dtab.p, tableStride, (const int *)dctx.p, (const int *)dslot.p, maxCtx, nullptr));
    } else {
        int sum = 0;
        for (int b = 0; b < batch_size; ++b) sum += token_lens[b];
        if (sum != total) {
            printf("invokeAttention: token_lens sum to %d, query_shape[0] is %d\n", sum, total);
            exit(-1);
        }
        CK(xfthip_paged_attention_prefill(dout.p, dq.p, dk.p, dv.p, qHeads, kvHeads, headSize, q_stride, kv_stride, oStride, scale, batch_size,
                token_lens, kc, vc, blockNum, blockSize, (const int *)dslot.p, nullptr));
    }
    CK(xfthip_memcpy_d2h(output, dout.p, (size_t)rows * oStride * 2, nullptr));
    // the host copies of the caches get the new rows too
    for (int r = 0; r < rows; ++r) {
        const int slot = slot_mapping[r];
        if (slot < 0 || slot >= blockNum * blockSize) continue;
        memcpy((uint16_t *)const_cast<void *>(kcache) + (size_t)slot * rowElems, (const uint16_t *)key + (size_t)r * kv_stride, rowElems * 2);
        memcpy((uint16_t *)const_cast<void *>(vcache) + (size_t)slot * rowElems, (const uint16_t *)value + (size_t)r * kv_stride, rowElems * 2);
    }
}

void invokeAttentionLLaMA(DataType dt, int batchSize, int inputSeqLen, int attHeadDim, int attHeadNum, int kvHeadNum,
        int maxPositions, int maxPosEmbed, int pastSeqLen, int currentSeqLen, int step, int hiddenSize, void *output,
        int outputStride, const void *input, int inputStride, const void *queryWeight, const void *keyWeight,
        const void *valueWeight, const void *attnOutWeight, const float *queryBias, const float *keyBias,
        const float *valueBias, const float *attnOutBias) {
    static std::mutex mutex;
    std::lock_guard<std::mutex> lock(mutex);
    (void)currentSeqLen; (void)step;
    const int kind = kind_of(dt);
    if (kind < 0) return;
    ensure_init();

    static std::unordered_map<std::string, Entry> hub;
    std::stringstream key;
    key << queryWeight << "_" << keyWeight << "_" << valueWeight << "_" << attnOutWeight << "_" << queryBias << "_" << keyBias << "_"
        << valueBias << "_" << dt << "_" << attHeadDim << "_" << attHeadNum << "_" << kvHeadNum;
    Entry &e = hub[key.str()];
    if (!e.hasAttn) {
        const int qCols = attHeadNum * attHeadDim, kvCols = kvHeadNum * attHeadDim;
        auto qkv = concat_qkv((const float *)queryWeight, (const float *)keyWeight, (const float *)valueWeight, hiddenSize, qCols, kvCols);
        e.qkv = make_weight(kind, hiddenSize, qCols + 2 * kvCols, qkv.data(), XFTHIP_WF_NONE);
        e.o = make_weight(kind, qCols, hiddenSize, (const float *)attnOutWeight, XFTHIP_WF_NONE);
        e.qkvBias = concat_bias(queryBias, keyBias, valueBias, qCols, kvCols);
        if (attnOutBias) e.oBias.assign(attnOutBias, attnOutBias + hiddenSize);
        e.hasAttn = true;
        // the attention-only context of the reference has intermediate size 1 (attention.cpp:88-90);
        // the scratch here needs a multiple of 16
        e.cfg = xfthip_model_config {1, hiddenSize, 16, attHeadNum, kvHeadNum, attHeadDim, 0, batchSize, maxPositions,
                batchSize * inputSeqLen, maxPosEmbed, 10000, XFTHIP_FP16, 1e-6f};
        printf(">> create llama_attention_key: %s\n", key.str().c_str());
    }
    fit_model(e, batchSize, batchSize * inputSeqLen, maxPositions, maxPosEmbed);
    run_rows(input, inputStride, output, outputStride, batchSize * inputSeqLen, hiddenSize, [&](const float *di, float *dop) {
        CK(xfthip_model_attention_forward(e.model, 0, di, hiddenSize, dop, hiddenSize, batchSize, inputSeqLen, pastSeqLen, 0, nullptr));
    });
}

void invokeMLPLLaMA(DataType dt, ActivationType at, int numTokens, int hiddenSize, int intermediateSize, void *output,
        int outputStride, const void *input, int inputStride, const void *gateWeight, const void *upWeight,
        const void *downWeight) {
    static std::mutex mutex;
    std::lock_guard<std::mutex> lock(mutex);
    const int kind = kind_of(dt);
    if (kind < 0) return;
    if (at != ActivationType::SILU && at != ActivationType::SWIGLU) {
        printf(">> unsupported activation type\n");
        return;
    }
    ensure_init();

    static std::unordered_map<std::string, Entry> hub;
    std::stringstream key;
    key << gateWeight << "_" << upWeight << "_" << downWeight << "_" << dt << "_" << at;
    Entry &e = hub[key.str()];
    if (!e.hasMlp) {
        auto gu = concat_gateup((const float *)gateWeight, (const float *)upWeight, hiddenSize, intermediateSize);
        e.gateup = make_weight(kind, hiddenSize, 2 * intermediateSize, gu.data(), kind == XFTHIP_W_W8A8 ? XFTHIP_WF_NONE : XFTHIP_WF_GATEUP);
        e.down = make_weight(kind, intermediateSize, hiddenSize, (const float *)downWeight, XFTHIP_WF_NONE);
        e.hasMlp = true;
        // head geometry is irrelevant to the MLP block; one 128-wide head keeps the scratch small
        e.cfg = xfthip_model_config {1, hiddenSize, intermediateSize, 1, 1, 128, 0, 1, 32, numTokens, 32, 10000, XFTHIP_FP16, 1e-6f};
        printf(">> create llama_mlp_key: %s\n", key.str().c_str());
    }
    fit_model(e, 1, numTokens, 32, 32);
    run_rows(input, inputStride, output, outputStride, numTokens, hiddenSize, [&](const float *di, float *dop) {
        CK(xfthip_model_mlp_forward(e.model, 0, di, hiddenSize, dop, hiddenSize, numTokens, 0, nullptr));
    });
}

void invokeRmsNorm(DataType dt, void *output, const void *input, const void *weight, int rows, int cols, int iStride,
        int oStride, float epsilon) {
    if (dt != DataType::fp32 && dt != DataType::bf16) return; // fp16 activations are not offered by this build
    ensure_init();
    if (iStride == -1) iStride = cols;
    if (oStride == -1) oStride = cols;
    const int et = dt == DataType::fp32 ? XFTHIP_F32 : XFTHIP_BF16;
    const size_t esz = dt == DataType::fp32 ? 4 : 2;
    // weight has the element type of dt (src/kernels/rmsnorm_kernels.cpp:166-180); the kernel wants fp32
    std::vector<float> w(cols);
    for (int i = 0; i < cols; ++i) w[i] = dt == DataType::fp32 ? ((const float *)weight)[i] : from_bf16(((const uint16_t *)weight)[i]);
    void *di = nullptr, *dop = nullptr, *dw = nullptr;
    CK(xfthip_malloc(&di, (size_t)rows * iStride * esz));
    CK(xfthip_malloc(&dop, (size_t)rows * oStride * esz));
    CK(xfthip_malloc(&dw, (size_t)cols * 4));
    CK(xfthip_memcpy_h2d(di, input, ((size_t)(rows - 1) * iStride + cols) * esz, nullptr));
    CK(xfthip_memcpy_h2d(dop, output, ((size_t)(rows - 1) * oStride + cols) * esz, nullptr)); // keep the gaps between rows
    CK(xfthip_memcpy_h2d(dw, w.data(), (size_t)cols * 4, nullptr));
    CK(xfthip_rmsnorm(dop, et, di, et, (const float *)dw, rows, cols, iStride, oStride, epsilon, nullptr));
    CK(xfthip_memcpy_d2h(output, dop, ((size_t)(rows - 1) * oStride + cols) * esz, nullptr));
    xfthip_free(di);
    xfthip_free(dop);
    xfthip_free(dw);
}

void invokeLayerNorm(DataType dt, void *output, const void *input, const void *gamma, const void *beta, int rows, int cols,
        int iStride, int oStride, float epsilon) {
    // fp32 and bf16 buffers; fp16 activations are not offered by this build (the reference's dispatch has no
    // else-branch either: an unknown dt is a silent no-op, layernorm_kernels.cpp:148-160)
    if (dt != DataType::fp32 && dt != DataType::bf16) return;
    ensure_init();
    if (iStride == -1) iStride = cols;
    if (oStride == -1) oStride = cols;
    const int et = dt == DataType::fp32 ? XFTHIP_F32 : XFTHIP_BF16;
    const size_t esz = dt == DataType::fp32 ? 4 : 2;
    // gamma and beta have the element type of dt; the kernel wants fp32
    std::vector<float> gb((size_t)2 * cols);
    for (int i = 0; i < cols; ++i) {
        gb[i] = dt == DataType::fp32 ? ((const float *)gamma)[i] : from_bf16(((const uint16_t *)gamma)[i]);
        gb[cols + i] = dt == DataType::fp32 ? ((const float *)beta)[i] : from_bf16(((const uint16_t *)beta)[i]);
    }
    void *di = nullptr, *dop = nullptr, *dw = nullptr;
    CK(xfthip_malloc(&di, (size_t)rows * iStride * esz));
    CK(xfthip_malloc(&dop, (size_t)rows * oStride * esz));
    CK(xfthip_malloc(&dw, gb.size() * 4));
    CK(xfthip_memcpy_h2d(di, input, ((size_t)(rows - 1) * iStride + cols) * esz, nullptr));
    CK(xfthip_memcpy_h2d(dop, output, ((size_t)(rows - 1) * oStride + cols) * esz, nullptr)); // keep the gaps between rows
    CK(xfthip_memcpy_h2d(dw, gb.data(), gb.size() * 4, nullptr));
    CK(xfthip_layernorm(dop, et, di, et, (const float *)dw, (const float *)dw + cols, rows, cols, iStride, oStride, epsilon, nullptr));
    CK(xfthip_memcpy_d2h(output, dop, ((size_t)(rows - 1) * oStride + cols) * esz, nullptr));
    xfthip_free(di);
    xfthip_free(dop);
    xfthip_free(dw);
}

void invokeRotaryEmbedding(DataType dt, const int64_t *positionIds, void *query, void *key, const void *embCos,
        const void *embSin, const int dim, const int qStride, const int kStride, const int numTokens, const int headNum,
        const int headSize, const int numKvHeads) {
    // the reference treats dt == fp16 buffers as fp32 (src/layers/rotary_embedding_api.cpp:87-96); kept
    if (dt != DataType::bf16 && dt != DataType::fp16 && dt != DataType::fp32) return;
    if (dim != headSize) {
        printf("Incorrect shape, rot_dim is not the head size.\n");
        exit(-1);
    }
    ensure_init();
    const bool isbf = dt == DataType::bf16;
    const int et = isbf ? XFTHIP_BF16 : XFTHIP_F32;
    const size_t esz = isbf ? 2 : 4;
    const int kvHeads = numKvHeads > 0 ? numKvHeads : headNum;
    int maxPos = 0;
    std::vector<int> pos(numTokens);
    for (int i = 0; i < numTokens; ++i) {
        pos[i] = (int)positionIds[i];
        if (pos[i] > maxPos) maxPos = pos[i];
    }
    // tables arrive as [maxPosition, dim] in the element type of dt; the kernel takes fp32
    const size_t tn = (size_t)(maxPos + 1) * dim;
    std::vector<float> c(tn), s(tn);
    for (size_t i = 0; i < tn; ++i) {
        c[i] = isbf ? from_bf16(((const uint16_t *)embCos)[i]) : ((const float *)embCos)[i];
        s[i] = isbf ? from_bf16(((const uint16_t *)embSin)[i]) : ((const float *)embSin)[i];
    }
    const size_t qBytes = ((size_t)(numTokens - 1) * qStride + (size_t)headNum * headSize) * esz;
    const size_t kBytes = ((size_t)(numTokens - 1) * kStride + (size_t)kvHeads * headSize) * esz;
    void *dq = nullptr, *dk = nullptr, *dc = nullptr, *ds = nullptr, *dp = nullptr;
    CK(xfthip_malloc(&dq, qBytes));
    CK(xfthip_malloc(&dk, kBytes));
    CK(xfthip_malloc(&dc, tn * 4));
    CK(xfthip_malloc(&ds, tn * 4));
    CK(xfthip_malloc(&dp, (size_t)numTokens * 4));
    CK(xfthip_memcpy_h2d(dq, query, qBytes, nullptr));
    CK(xfthip_memcpy_h2d(dk, key, kBytes, nullptr));
    CK(xfthip_memcpy_h2d(dc, c.data(), tn * 4, nullptr));
    CK(xfthip_memcpy_h2d(ds, s.data(), tn * 4, nullptr));
    CK(xfthip_memcpy_h2d(dp, pos.data(), (size_t)numTokens * 4, nullptr));
    CK(xfthip_rotary_embedding_full(et, (const int *)dp, dq, dk, (const float *)dc, (const float *)ds, dim, qStride, kStride,
            numTokens, headNum, headSize, kvHeads, nullptr));
    CK(xfthip_memcpy_d2h(query, dq, qBytes, nullptr));
    CK(xfthip_memcpy_d2h(key, dk, kBytes, nullptr));
    for (void *p : {dq, dk, dc, ds, dp}) xfthip_free(p);
}


void invokeGemm(DataType dt, bool transA, bool transB, int M, int N, int K, float alpha, void *A, int lda, void *B, float beta, void *C,
        int ldc, void *bias, void *res, int ldres) {
    // the reference accepts bias / res but never reads them (src/utils/matmul_helper.h:63-101)
    (void)bias; (void)res; (void)ldres;
    if (dt != DataType::bf16 && dt != DataType::fp16) {
        printf(">> invokeGemm: only bf16 and fp16 are offered (as in the reference, src/kernels/gemm_kernel_ext.cpp:503-517)\n");
        return;
    }
    ensure_init();
    const bool half = dt == DataType::fp16;
    const uint16_t *a = (const uint16_t *)A, *b = (const uint16_t *)B;
    auto a_at = [&](int m, int k) { return transA ? a[(size_t)k * M + m] : a[(size_t)m * lda + k]; };
    auto b_at = [&](int k, int n) { return transB ? b[(size_t)n * K + k] : b[(size_t)k * N + n]; };
    // The device GEMM multiplies bf16 by bf16.  An fp16 value (11 significant bits) is the exact sum of
    // two bf16 values hi + lo, so the fp16 product runs as one bf16 GEMM over a tripled k extent:
    // [Ah | Ah | Al] x [Bh ; Bl ; Bh] = Ah Bh + Ah Bl + Al Bh (the dropped Al Bl term is below 2^-16 of
    // the product).  bf16 runs as it is.
    const int parts = half ? 3 : 1;
    const int Kp = (K + 7) / 8 * 8;
    auto split = [&](uint16_t h, uint16_t &hi, uint16_t &lo) {
        const float f = from_fp16(h);
        hi = to_bf16(f);
        lo = to_bf16(f - from_bf16(hi));
    };
    std::vector<uint16_t> am((size_t)M * Kp * parts, 0), bp((size_t)Kp * parts * N, 0);
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            uint16_t *row = &am[(size_t)m * Kp * parts];
            if (half) {
                uint16_t hi, lo;
                split(a_at(m, k), hi, lo);
                row[k] = hi, row[Kp + k] = hi, row[2 * Kp + k] = lo;
            } else {
                row[k] = a_at(m, k);
            }
        }
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) {
            if (half) {
                uint16_t hi, lo;
                split(b_at(k, n), hi, lo);
                bp[(size_t)k * N + n] = hi, bp[((size_t)Kp + k) * N + n] = lo, bp[((size_t)2 * Kp + k) * N + n] = hi;
            } else {
                bp[(size_t)k * N + n] = b_at(k, n);
            }
        }
    xfthip_weight_t w = nullptr;
    CK(xfthip_weight_create(XFTHIP_W_BF16, Kp * parts, N, bp.data(), nullptr, nullptr, XFTHIP_WF_NONE, &w));
    void *da = nullptr, *dc = nullptr;
    CK(xfthip_malloc(&da, am.size() * 2));
    CK(xfthip_malloc(&dc, (size_t)M * N * 4));
    CK(xfthip_memcpy_h2d(da, am.data(), am.size() * 2, nullptr));
    CK(xfthip_gemm(w, M, da, Kp * parts, dc, N, XFTHIP_F32, XFTHIP_EPI_NONE, nullptr, nullptr, 0, XFTHIP_F32, 1.0f, nullptr));
    std::vector<float> acc((size_t)M * N);
    CK(xfthip_memcpy_d2h(acc.data(), dc, acc.size() * 4, nullptr));
    uint16_t *c = (uint16_t *)C;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float v = alpha * acc[(size_t)m * N + n];
            if (beta != 0.0f) v += beta * (half ? from_fp16(c[(size_t)m * ldc + n]) : from_bf16(c[(size_t)m * ldc + n]));
            c[(size_t)m * ldc + n] = half ? to_fp16(v) : to_bf16(v);
        }
    xfthip_free(da);
    xfthip_free(dc);
    xfthip_weight_destroy(w);
}

} // namespace xft
