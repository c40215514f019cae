// xft::invokeAttention and xft::invokeAttentionLLaMA, source-compatible with the reference's
// include/layers_attention.h:52-65.
//
// invokeAttention: attention over a block-paged BF16 KV cache for continuous batching (bf16 only, as in
// the reference: any other dt prints an error and exits).  All pointers are host memory.
//   query [total_tokens, q_stride], key / value [total_tokens, kv_stride], output
//   [total_tokens, query_head_num * head_size], all bf16; query_shape = {total_tokens, query_head_num,
//   head_size}, kv_shape = {total_tokens, kv_head_num, head_size}; kcache / vcache
//   [block_num, block_size, kv_head_num, head_size] bf16 with kvcache_shape naming those four sizes.
//   is_prefill = false: one new token per sequence (total_tokens = batch_size); key / value row b is
//   written to slot slot_mapping[b] (slot = block * block_size + row), then query row b attends to the
//   context_lens[b] + 1 tokens that row b of block_tables maps.  block_tables is a dense
//   [batch_size, max(block_nums)] array; block_nums[b] entries of row b are valid and must cover
//   context_lens[b] + 1 tokens.
//   is_prefill = true: token_lens[b] new tokens per sequence, back to back; causal self-attention per
//   sequence, and every token's key / value row goes to slot_mapping[token] (one entry per token).
//   The callee keeps a device copy of each cache it has seen (keyed by the host address; uploaded on
//   first sight) and writes the new rows to both copies: other writers of the host cache are not observed.
// Departures from the reference's text (src/kernels/attention_kernels.cpp:24-157), which has no test:
// query / key / value row b is used for sequence b (the reference reads row 0 for every sequence), the KV
// head of query head i is i / (query_head_num / kv_head_num) (the reference uses i), the table row stride
// is max(block_nums) (the reference derives it from the largest context without the new token) and
// prefill stores every token (the reference's store closures are marked "TODO: debug and fix").
//
// invokeAttentionLLaMA:
// output = Attention(input) * Wo + bias + input (no input norm), fp32 host buffers
// [batchSize*inputSeqLen, stride].  query/key/value weights are the three column blocks of one
// fp32 [hiddenSize, (attHeadNum + 2*kvHeadNum) * attHeadDim] host matrix (row stride = that
// width), attnOutWeight is [attHeadNum*attHeadDim, hiddenSize].  The KV cache (FP16) belongs to
// the callee and carries over between calls: pastSeqLen / step are supplied by the caller.
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeAttention(DataType dt, void *output, const void *query, const void *key, const void *value, int *query_shape,
        int *kv_shape, const int q_stride, const int kv_stride, const float scale, const int batch_size,
        const int *token_lens, const void *kcache, const void *vcache, int *kvcache_shape, int *block_tables,
        int *block_nums, int *context_lens, int layer_id, bool is_prefill, int *slot_mapping);

void invokeAttentionLLaMA(DataType dt, int batchSize, int inputSeqLen, int attHeadDim, int attHeadNum, int kvHeadNum,
        int maxPositions, int maxPosEmbed, int pastSeqLen, int currentSeqLen, int step, int hiddenSize, void *output,
        int outputStride, const void *input, int inputStride, const void *queryWeight, const void *keyWeight,
        const void *valueWeight, const void *attnOutWeight, const float *queryBias = nullptr,
        const float *keyBias = nullptr, const float *valueBias = nullptr, const float *attnOutBias = nullptr);

} // namespace xft
