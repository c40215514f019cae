// Mixtral-style sparse MLP: router GEMM, top-2 selection with a 2-way softmax, per-expert gather,
// SwiGLU MLP on the gathered rows and weighted scatter-add.  Replaces MixtralMLP::forward,
// selectTop2Experts, gatherInput and scatterOutput (reference src/layers/mlp_mixtral.h:29-291).
// Experts run one after another in ascending order, as the reference's loop does, so every
// token's two contributions are added in a fixed order.
#include <vector>

#include "common.h"
#include "qgemm.h"

namespace xfthip {

// logits[t][e] = sum_k xn[t][k] * Wr[k][e]; one wave per token, fp32 router weights
// (GateTypeSelector: fp32 for quantised weight types, src/utils/type_selector.h:93-111)
template <int E>
__global__ __launch_bounds__(64) void router_kernel(const uint16_t *__restrict__ xn, int ld, const float *__restrict__ Wr,
        float *__restrict__ logits, int hidden) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.0f;
    for (int k = lane; k < hidden; k += 64) {
        const float x = bf16_to_f32(xn[(size_t)t * ld + k]);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] = fmaf(x, Wr[(size_t)k * E + e], acc[e]);
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc[e] += __shfl_xor(acc[e], off, 64);
    }
    if (lane == 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) logits[(size_t)t * E + e] = acc[e];
    }
}

// strict '>' scan: the lower index wins ties (mlp_mixtral.h:262-283); weights = softmax over the
// two selected logits (:221-259)
__global__ void top2_kernel(const float *__restrict__ logits, int M, int E, int *__restrict__ sel, float *__restrict__ w) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= M) return;
    float max1 = -INFINITY, max2 = -INFINITY;
    int idx1 = -1, idx2 = -1;
    for (int j = 0; j < E; ++j) {
        const float v = logits[(size_t)t * E + j];
        if (v > max1) {
            max2 = max1;
            idx2 = idx1;
            max1 = v;
            idx1 = j;
        } else if (v > max2) {
            max2 = v;
            idx2 = j;
        }
    }
    const float e1 = 1.0f, e2 = fast_exp(max2 - max1); // relative to the larger of the two
    sel[2 * t] = idx1;
    sel[2 * t + 1] = idx2;
    w[2 * t] = e1 / (e1 + e2);
    w[2 * t + 1] = e2 / (e1 + e2);
}

// Per-expert token lists in ascending token order, in one workgroup: wave e collects expert e's tokens 64 at
// a time (ballot + prefix count), then the lists are laid back to back (expert 0's rows first) and every
// (token, choice) learns the row of the gathered matrix that holds its copy:
//   counts[e], offsets[e] (first row of expert e), row_token[g] / row_weight[g] for the 2 M gathered rows,
//   slot_row[2 t + s] = row of token t's s-th choice, gemm_rows[9 e ..] = the row records of expert e's GEMMs.
// blockDim.x = 64 * E; rank[] is scratch of 2 M ints.
__global__ __launch_bounds__(512) void build_lists_kernel(const int *__restrict__ sel, const float *__restrict__ w, int M, int E,
        int *__restrict__ counts, int *__restrict__ offsets, int *__restrict__ row_token, float *__restrict__ row_weight,
        int *__restrict__ slot_row, int *__restrict__ rank, int *__restrict__ gemm_rows) {
    __shared__ int s_count[8], s_off[8];
    const int e = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int n = 0;
    for (int t0 = 0; t0 < M; t0 += 64) {
        const int t = t0 + lane;
        int slot = -1;
        if (t < M) slot = sel[2 * t] == e ? 0 : (sel[2 * t + 1] == e ? 1 : -1);
        const unsigned long long mask = __ballot(slot >= 0);
        if (slot >= 0) rank[2 * t + slot] = n + __popcll(mask & ((1ull << lane) - 1ull));
        n += __popcll(mask);
    }
    if (lane == 0) s_count[e] = n;
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        for (int i = 0; i < E; ++i) {
            s_off[i] = acc;
            counts[i] = s_count[i];
            offsets[i] = acc;
            // what the two GEMMs of expert i read instead of a host-side row count: {rows, first row of A, first
            // row of C}: gate/up reads its gathered rows and writes the shared hidden buffer from row 0, down
            // reads that buffer and writes the expert-output rows
            // (the launch that serves all experts at once keeps every expert's hidden rows: {rows, first, first})
            gemm_rows[9 * i + 0] = s_count[i], gemm_rows[9 * i + 1] = acc, gemm_rows[9 * i + 2] = 0;
            gemm_rows[9 * i + 3] = s_count[i], gemm_rows[9 * i + 4] = 0, gemm_rows[9 * i + 5] = acc;
            gemm_rows[9 * i + 6] = s_count[i], gemm_rows[9 * i + 7] = acc, gemm_rows[9 * i + 8] = acc;
            acc += s_count[i];
        }
    }
    __syncthreads();
    // A token whose logits are NaN (or all -inf) has fewer than two choices: top2_kernel leaves -1 there, no wave
    // ranked that choice, and it takes no row, as in the reference, whose loop over the experts never matches it
    // (mlp_mixtral.h:165-186).  The gathered rows past the last expert's stay defined (token 0, weight 0): the
    // gather runs over all 2 M rows.
    const int total = s_off[E - 1] + s_count[E - 1];
    for (int i = threadIdx.x; i < 2 * M; i += blockDim.x) {
        const int e_sel = sel[i];
        if (i >= total) row_token[i] = 0, row_weight[i] = 0.0f;
        if (e_sel < 0 || e_sel >= E) slot_row[i] = -1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * M; i += blockDim.x) {
        const int e_sel = sel[i];
        if (e_sel < 0 || e_sel >= E) continue;
        const int t = i >> 1, g = s_off[e_sel] + rank[i];
        slot_row[i] = g;
        row_token[g] = t;
        row_weight[g] = w[i];
    }
}

// gathered[g] = xn[row_token[g]], 16 bytes a thread; grid = rows
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint16_t *__restrict__ xn, int ld, const int *__restrict__ row_token,
        uint16_t *__restrict__ out, int hidden) {
    const int r = blockIdx.x;
    const uint4 *src = (const uint4 *)(xn + (size_t)row_token[r] * ld);
    uint4 *dst = (uint4 *)(out + (size_t)r * hidden);
    for (int c = threadIdx.x; c < hidden / 8; c += blockDim.x) dst[c] = src[c];
}

// out[t] += eo[row of choice] * weight, the lower expert index first: the order in which the reference's
// loop over the experts adds a token's two contributions (xft::addto: one fused multiply-add per element).
// grid = tokens
// The residual comes straight from the layer's input (`in`, which may be `out` itself: a thread reads an element
// before it writes it), so no copy of the input into the output runs first.
__global__ __launch_bounds__(256) void combine_kernel(float *out, int ld, const float *in, int in_ld, const float *__restrict__ eo,
        const int *__restrict__ sel, const int *__restrict__ slot_row, const float *__restrict__ w, int hidden, int wide) {
    const int t = blockIdx.x;
    const int first = sel[2 * t] < sel[2 * t + 1] ? 0 : 1;
    const int ga = slot_row[2 * t + first], gb = slot_row[2 * t + 1 - first];
    const float wa = w[2 * t + first], wb = w[2 * t + 1 - first];
    if (ga < 0 || gb < 0) {
        // a choice without an expert (NaN logits) contributes nothing; not the common case, kept simple
        const float *ea = eo + (size_t)(ga < 0 ? 0 : ga) * hidden, *eb = eo + (size_t)(gb < 0 ? 0 : gb) * hidden;
        for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
            float o = in[(size_t)t * in_ld + c];
            if (ga >= 0) o = fmaf(ea[c], wa, o);
            if (gb >= 0) o = fmaf(eb[c], wb, o);
            out[(size_t)t * ld + c] = o;
        }
        return;
    }
    if (wide) { // rows of out start on 16-byte boundaries
        const float4 *ea = (const float4 *)(eo + (size_t)ga * hidden), *eb = (const float4 *)(eo + (size_t)gb * hidden);
        float4 *dst = (float4 *)(out + (size_t)t * ld);
        const float4 *src = (const float4 *)(in + (size_t)t * in_ld);
        for (int c = threadIdx.x; c < hidden / 4; c += blockDim.x) {
            float4 o = src[c];
            const float4 a = ea[c], b = eb[c];
            o.x = fmaf(b.x, wb, fmaf(a.x, wa, o.x));
            o.y = fmaf(b.y, wb, fmaf(a.y, wa, o.y));
            o.z = fmaf(b.z, wb, fmaf(a.z, wa, o.z));
            o.w = fmaf(b.w, wb, fmaf(a.w, wa, o.w));
            dst[c] = o;
        }
    } else {
        const float *ea = eo + (size_t)ga * hidden, *eb = eo + (size_t)gb * hidden;
        float *dst = out + (size_t)t * ld;
        const float *src = in + (size_t)t * in_ld;
        for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = fmaf(eb[c], wb, fmaf(ea[c], wa, src[c]));
    }
}

__global__ void narrow_rows_kernel2(const float *__restrict__ in, int in_stride, uint16_t *__restrict__ out, int cols) {
    const float *row = in + (size_t)blockIdx.x * in_stride;
    uint16_t *orow = out + (size_t)blockIdx.x * cols;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) orow[c] = f32_to_bf16_ref(row[c]);
}

} // namespace xfthip

using namespace xfthip;

struct xfthip_moe {
    int hidden, inter, E, max_tokens;
    float *router = nullptr, *ln = nullptr;
    std::vector<xfthip_weight_t> gateup, down;
    uint16_t *xn = nullptr, *xg = nullptr, *h = nullptr;
    float *eo = nullptr, *logits = nullptr, *w = nullptr, *row_weight = nullptr;
    GroupWeight *group = nullptr; // device pointers of the experts' weights: [E] gate/up, [E] down
    int *sel = nullptr, *counts = nullptr, *row_token = nullptr, *slot_row = nullptr, *rank = nullptr; // counts: [E] counts, [E] offsets, [9 E] GEMM row records
    bool owns_workspace = true; // false: the per-call buffers belong to the object this one was created beside
};

extern "C" {

int xfthip_moe_top2(const float *logits, int M, int E, int *sel, float *weights, xfthip_stream_t stream) {
    XFT_REQUIRE(logits && sel && weights && M > 0 && E >= 2, "xfthip_moe_top2: bad argument");
    hipLaunchKernelGGL(top2_kernel, dim3((M + 255) / 256), dim3(256), 0, (hipStream_t)stream, logits, M, E, sel, weights);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_moe_create(int hidden, int intermediate, int experts, int max_tokens, const float *router_host, const float *ln_host,
        xfthip_moe_t *out) {
    XFT_REQUIRE(out && router_host, "xfthip_moe_create: null argument");
    XFT_REQUIRE(experts == 8, "xfthip_moe_create: %d experts unsupported (the router kernel is built for 8)", experts);
    XFT_REQUIRE(hidden > 0 && hidden % 8 == 0 && intermediate % 16 == 0 && max_tokens > 0, "xfthip_moe_create: bad sizes");
    xfthip_moe *m = new xfthip_moe();
    m->hidden = hidden;
    m->inter = intermediate;
    m->E = experts;
    m->max_tokens = max_tokens;
    m->gateup.assign(experts, nullptr);
    m->down.assign(experts, nullptr);
    const size_t T = max_tokens;
    // every token is gathered twice (its two experts): 2 T rows of activations and of expert outputs
    bool ok = hipMalloc((void **)&m->router, (size_t)hidden * experts * 4) == hipSuccess
            && hipMalloc((void **)&m->xn, T * hidden * 2) == hipSuccess && hipMalloc((void **)&m->xg, 2 * T * hidden * 2) == hipSuccess
            && hipMalloc((void **)&m->h, 2 * T * intermediate * 2) == hipSuccess && hipMalloc((void **)&m->eo, 2 * T * hidden * 4) == hipSuccess
            && hipMalloc((void **)&m->logits, T * experts * 4) == hipSuccess && hipMalloc((void **)&m->w, T * 2 * 4) == hipSuccess
            && hipMalloc((void **)&m->sel, T * 2 * 4) == hipSuccess && hipMalloc((void **)&m->counts, (2 + 9) * 64) == hipSuccess && hipMalloc((void **)&m->group, 2 * 64 * sizeof(GroupWeight)) == hipSuccess
            && hipMalloc((void **)&m->row_token, 2 * T * 4) == hipSuccess && hipMalloc((void **)&m->row_weight, 2 * T * 4) == hipSuccess
            && hipMalloc((void **)&m->slot_row, 2 * T * 4) == hipSuccess && hipMalloc((void **)&m->rank, 2 * T * 4) == hipSuccess;
    if (ok && ln_host) ok = hipMalloc((void **)&m->ln, (size_t)hidden * 4) == hipSuccess
            && hipMemcpy(m->ln, ln_host, (size_t)hidden * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (ok) ok = hipMemcpy(m->router, router_host, (size_t)hidden * experts * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (!ok) {
        set_error("xfthip_moe_create: allocation failed");
        xfthip_moe_destroy(m);
        return 1;
    }
    *out = m;
    return 0;
}

int xfthip_moe_create_beside(xfthip_moe_t first, const float *router_host, const float *ln_host, xfthip_moe_t *out) {
    XFT_REQUIRE(first && out && router_host, "xfthip_moe_create_beside: null argument");
    XFT_REQUIRE(first->owns_workspace, "xfthip_moe_create_beside: the first object must own its workspace");
    xfthip_moe *m = new xfthip_moe(*first);
    m->owns_workspace = false;
    m->router = nullptr, m->ln = nullptr, m->group = nullptr;
    m->gateup.assign(m->E, nullptr);
    m->down.assign(m->E, nullptr);
    bool ok = hipMalloc((void **)&m->router, (size_t)m->hidden * m->E * 4) == hipSuccess
            && hipMalloc((void **)&m->group, 2 * 64 * sizeof(GroupWeight)) == hipSuccess
            && hipMemcpy(m->router, router_host, (size_t)m->hidden * m->E * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (ok && ln_host) ok = hipMalloc((void **)&m->ln, (size_t)m->hidden * 4) == hipSuccess
            && hipMemcpy(m->ln, ln_host, (size_t)m->hidden * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (!ok) {
        set_error("xfthip_moe_create_beside: allocation failed");
        xfthip_moe_destroy(m);
        return 3;
    }
    *out = m;
    return 0;
}

int xfthip_moe_destroy(xfthip_moe_t m) {
    if (!m) return 0;
    void *own[] = {m->router, m->ln, m->group};
    void *workspace[] = {m->xn, m->xg, m->h, m->eo, m->logits, m->w, m->row_weight, m->sel, m->counts, m->row_token, m->slot_row, m->rank};
    for (void *b : own)
        if (b) (void)hipFree(b);
    if (m->owns_workspace)
        for (void *b : workspace)
            if (b) (void)hipFree(b);
    delete m;
    return 0;
}

int xfthip_moe_shape(xfthip_moe_t m, int *hidden, int *intermediate, int *experts, int *max_tokens) {
    XFT_REQUIRE(m, "xfthip_moe_shape: null argument");
    if (hidden) *hidden = m->hidden;
    if (intermediate) *intermediate = m->inter;
    if (experts) *experts = m->E;
    if (max_tokens) *max_tokens = m->max_tokens;
    return 0;
}

int xfthip_moe_set_expert(xfthip_moe_t m, int e, xfthip_weight_t gateup, xfthip_weight_t down) {
    XFT_REQUIRE(m && gateup && down && e >= 0 && e < m->E, "xfthip_moe_set_expert: bad argument");
    XFT_REQUIRE(gateup->pw.K == m->hidden && gateup->pw.N == 2 * m->inter && (gateup->pw.flags & XFTHIP_WF_GATEUP),
            "xfthip_moe_set_expert: gate/up weight must be [%d,%d] created with XFTHIP_WF_GATEUP", m->hidden, 2 * m->inter);
    XFT_REQUIRE(down->pw.K == m->inter && down->pw.N == m->hidden, "xfthip_moe_set_expert: down weight must be [%d,%d]", m->inter, m->hidden);
    m->gateup[e] = gateup;
    m->down[e] = down;
    const GroupWeight g = {gateup->pw.packed, gateup->pw.scale, gateup->pw.zero}, d = {down->pw.packed, down->pw.scale, down->pw.zero};
    XFT_CHECK_HIP(hipMemcpy(m->group + e, &g, sizeof(g), hipMemcpyHostToDevice));
    XFT_CHECK_HIP(hipMemcpy(m->group + m->E + e, &d, sizeof(d), hipMemcpyHostToDevice));
    return 0;
}

int xfthip_moe_forward(xfthip_moe_t m, const float *x_in, int in_stride, float *x_out, int out_stride, int tokens, int do_norm,
        const float *logits_override, int *sel_host_out, float *w_host_out, xfthip_stream_t stream) {
    XFT_REQUIRE(m && x_in && x_out, "xfthip_moe_forward: null argument");
    XFT_REQUIRE(tokens > 0 && tokens <= m->max_tokens, "xfthip_moe_forward: %d tokens exceed max_tokens %d", tokens, m->max_tokens);
    XFT_REQUIRE(in_stride >= m->hidden && out_stride >= m->hidden, "xfthip_moe_forward: stride smaller than hidden");
    XFT_REQUIRE(!do_norm || m->ln, "xfthip_moe_forward: no norm weight was given at creation");
    for (int e = 0; e < m->E; ++e) XFT_REQUIRE(m->gateup[e] && m->down[e], "xfthip_moe_forward: expert %d has no weights", e);
    hipStream_t st = (hipStream_t)stream;
    const int T = tokens, H = m->hidden;
    // residual (mlp_mixtral.h:116-121: the output starts as a copy of the input): combine_kernel reads it from x_in
    if (do_norm) {
        if (int rc = xfthip_rmsnorm(m->xn, XFTHIP_BF16, x_in, XFTHIP_F32, m->ln, T, H, in_stride, H, 1e-6f, st)) return rc;
    } else {
        hipLaunchKernelGGL(narrow_rows_kernel2, dim3(T), dim3(256), 0, st, x_in, in_stride, m->xn, H);
    }
    const float *logits = logits_override;
    if (!logits) {
        hipLaunchKernelGGL(router_kernel<8>, dim3(T), dim3(64), 0, st, m->xn, H, m->router, m->logits, H);
        logits = m->logits;
    }
    if (int rc = xfthip_moe_top2(logits, T, m->E, m->sel, m->w, st)) return rc;
    int *gemm_rows = m->counts + 2 * m->E;
    hipLaunchKernelGGL(build_lists_kernel, dim3(1), dim3(64 * m->E), 0, st, m->sel, m->w, T, m->E, m->counts, m->counts + m->E, m->row_token,
            m->row_weight, m->slot_row, m->rank, gemm_rows);
    hipLaunchKernelGGL(gather_rows_kernel, dim3(2 * T), dim3(256), 0, st, m->xn, H, m->row_token, m->xg, H);
    XFT_CHECK_HIP(hipGetLastError());
    if (sel_host_out || w_host_out) {
        XFT_CHECK_HIP(hipStreamSynchronize(st));
        if (sel_host_out) XFT_CHECK_HIP(hipMemcpy(sel_host_out, m->sel, (size_t)T * 2 * 4, hipMemcpyDeviceToHost));
        if (w_host_out) XFT_CHECK_HIP(hipMemcpy(w_host_out, m->w, (size_t)T * 2 * 4, hipMemcpyDeviceToHost));
    }
    // The host never learns how many rows an expert got: the GEMMs read row counts and row offsets from the
    // records build_lists_kernel left in device memory, and nothing here synchronises, so the layer can be
    // captured into a graph.  With experts of one kind, one launch serves the gate/up projections of all experts and
    // one their down projections (up to 32 tokens: the few-row kernel, a grid row an expert, experts without rows
    // leave at once; more: the tiled kernel, row blocks numbered across the experts); their workgroups run side by
    // side instead of one expert after another.  Otherwise every expert's two GEMMs are launched for up to T rows, in
    // the form for the 2 T / E rows an expert gets on average, and workgroups past the count leave at once.
    bool uniform = true;
    for (int e = 1; e < m->E && uniform; ++e) {
        const PackedWeight &g0 = m->gateup[0]->pw, &g = m->gateup[e]->pw, &d0 = m->down[0]->pw, &d = m->down[e]->pw;
        uniform = g.kind == g0.kind && g.flags == g0.flags && (g.zero != nullptr) == (g0.zero != nullptr) && d.kind == d0.kind
                && d.flags == d0.flags && (d.zero != nullptr) == (d0.zero != nullptr);
    }
    // (the few-row form of the grouped launch has no K-tail variant: a K that is not a whole number of weight
    // tiles goes expert by expert)
    if (T <= 32) {
        const PackedWeight &g0 = m->gateup[0]->pw, &d0 = m->down[0]->pw;
        uniform = uniform && g0.KT * ktile_of(g0.kind) == g0.K && d0.KT * ktile_of(d0.kind) == d0.K;
    }
    if (uniform && m->gateup[0]->pw.kind != XFTHIP_W_W8A8 && m->down[0]->pw.kind != XFTHIP_W_W8A8) {
        if (int rc = gemm_grouped_rows_dev(m->gateup.data(), m->E, m->group, 2 * T, T, gemm_rows + 6, 9, m->xg, H, m->h, m->inter, XFTHIP_BF16, st))
            return rc;
        if (int rc = gemm_grouped_rows_dev(m->down.data(), m->E, m->group + m->E, 2 * T, T, gemm_rows + 6, 9, m->h, m->inter, m->eo, H, XFTHIP_F32, st))
            return rc;
    } else {
        const int hint = (2 * T + m->E - 1) / m->E;
        for (int e = 0; e < m->E; ++e) {
            if (int rc = gemm_rows_dev(m->gateup[e], T, hint, gemm_rows + 9 * e, m->xg, H, m->h, m->inter, XFTHIP_BF16, st)) return rc;
            if (int rc = gemm_rows_dev(m->down[e], T, hint, gemm_rows + 9 * e + 3, m->h, m->inter, m->eo, H, XFTHIP_F32, st)) return rc;
        }
    }
    const int wide = (((size_t)x_out | ((size_t)out_stride * 4) | (size_t)x_in | ((size_t)in_stride * 4)) & 15) == 0 && H % 4 == 0;
    hipLaunchKernelGGL(combine_kernel, dim3(T), dim3(256), 0, st, x_out, out_stride, x_in, in_stride, m->eo, m->sel, m->slot_row, m->w, H, wide);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

} // extern "C"
