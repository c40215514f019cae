// Parameter block shared by the weight-only GEMM kernels and their C-ABI entry points.
#pragma once
#include "common.h"
#include "kvcache.h"

namespace xfthip {

struct GroupWeight { // one weight of a grouped launch, in device memory
    const uint8_t *packed;
    const float *scale;
    const float *zero;
};

struct SkinnyParams {
    const uint8_t *packed;
    const float *scale;
    const float *zero;
    int KT, NTILES, K, N, M;
    const uint16_t *A; // bf16
    int lda;
    void *C;
    int ldc, c_dtype;
    int epi;
    const float *bias;
    const void *res;
    int ldres, res_dtype;
    float gamma;
    int gateup; // 1: combine tile pairs as silu(gate)*up, N counts cat columns
    int nblocks; // column blocks of the launch (set by the launcher)
    // K split of the M > 32 kernel (few rows against few columns and a deep K): workgroup row blockIdx.y
    // multiplies k tiles [y * split_ktiles, (y + 1) * split_ktiles) and writes its scaled partial result as
    // fp32 [M][N] into split_part + y * M * N; a second kernel adds the parts in order and applies the epilogue
    int ksplit, split_ktiles;
    float *split_part;
    // Row count known on the device only (the experts of a sparse MLP): when rows_dev is set the kernels read
    // {rows, first row of A, first row of C} from it, M is only the upper bound that sizes the grid, and m_hint
    // (0 = M) is the row count the host expects, used where it chooses between forms.  No residual epilogues.
    const int *rows_dev;
    int m_hint;
    // Several weights of one shape and kind behind one launch (M > 32 kernel only): weight e multiplies the rows
    // that record e of rows_dev (records rows_stride ints apart) names; M bounds the sum of their rows, and their
    // rows of C must tile [0, sum of rows) without gaps.
    const GroupWeight *group;
    int group_n, rows_stride;

    // ---- fusions of the decode step (M <= 4, skinny kernel only) ----
    // RMSNorm prologue: when norm_x is set, A is ignored and every workgroup normalises the M rows
    // of norm_x (fp32, row pitch ldx) with norm_w / norm_eps into LDS itself (same arithmetic as
    // the rmsnorm kernel, bf16 result) while its first weight tiles are in flight.
    const float *norm_x;
    int ldx;
    const float *norm_w;
    float norm_eps;
    // RoPE + cache append epilogue of the QKV projection (one new token per sequence, FP16 cache):
    // column tiles are paired (d, d + 64) within a head, the rotated query goes to C as bf16
    // (row pitch ldc, q_heads * 128 columns), rotated keys and the values go to the cache at
    // position pos_dev[m] (or pos_host when pos_dev is null).  The tables hold 64 entries a row.
    int rope;
    const float *cosT, *sinT;
    const int *pos_dev;
    int pos_host;
    int qH, kvH;
    KvView kv;
};

int qgemm_skinny(const PackedWeight &pw, const SkinnyParams &p, hipStream_t stream); // M <= 32
bool skinny_can_fuse_norm(const PackedWeight &pw, int M); // may SkinnyParams::norm_x be used
int qgemm_mfma(const PackedWeight &pw, const SkinnyParams &p, hipStream_t stream); // any M, built for M > 32
// the K-split workspace of qgemm_mfma launches on `stream` (allocated on the stream's first call: before a capture, say)
int qgemm_split_reserve(hipStream_t stream, float **out = nullptr);
// xfthip_gemm / xfthip_gemm_gateup_silu (by the weight's flag) with the row count in device memory: rows_dev =
// {rows, first row of A, first row of C}, at most m_max rows, about m_hint expected; plain epilogue only
int gemm_rows_dev(xfthip_weight_t w, int m_max, int m_hint, const int *rows_dev, const void *A, int lda, void *C, int ldc, int c_dtype,
        hipStream_t stream);

// The same for n_group weights of one shape behind one launch: table_dev holds their device pointers, record e
// of rows_dev (rows_stride ints apart) the rows of weight e; rows_max bounds the sum of the rows, rows_each_max the
// rows of one weight (up to 32 of those: the few-row kernel, one grid row a weight; more: the tiled kernel, row
// blocks numbered across the weights); the weights' rows of C tile [0, sum of rows).
int gemm_grouped_rows_dev(const xfthip_weight_t *w, int n_group, const GroupWeight *table_dev, int rows_max, int rows_each_max,
        const int *rows_dev, int rows_stride, const void *A, int lda, void *C, int ldc, int c_dtype, hipStream_t stream);

int gemm_w8a8_from_bf16(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, hipStream_t stream);

} // namespace xfthip
