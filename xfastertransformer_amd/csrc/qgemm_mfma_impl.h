// Kernel template of the dequant-fused weight-only GEMM for many activation rows (M > 32), the
// prefill shape.  Included by one translation unit per weight kind (qgemm_mfma_*.hip) so that
// the instantiations compile in parallel.
// Replaces MMHelper::compute* (reference src/utils/matmul_helper.h:565-1705) at large M, where
// the reference switches to AMX (oneDNN) kernels.  MFMA-bound.
//
// A workgroup of 4 wavefronts computes a (4*WN*32 columns) x (WM*32 rows) output tile.  Each
// wave owns WN column tiles and streams their packed codes from global memory straight into
// registers (the same 1-KiB tile layout the M <= 32 kernel uses: a 128-bit load per lane becomes
// MFMA "B" operands after widening), so weights never pass through LDS.  The activation rows are
// shared by the 4 waves: staged through three padded LDS tiles and read back as 128-bit "A"
// operands.  The k loop is a three-stage pipeline (weights two tiles ahead in registers,
// activations four tiles ahead in registers and two in LDS) whose memory instructions are spread
// over the MFMAs of a step; the widening of each operand runs one MFMA group ahead of its use.
// Scale / zero-point / bias / activation / residual are applied in the epilogue.
#pragma once
#include <type_traits>

#include "qgemm.h"

namespace xfthip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// f32_to_bf16_ref() as selects (bf16_convert.h): the same bits for every input
__device__ inline uint32_t f32_to_bf16_sel(float f) { return f32_bits_to_bf16_sel(__float_as_uint(f)); }

union MFrag {
    bf16x8 v;
    uint32_t u[4];
    u32x4 q;
};

__device__ inline uint32_t pack_hi16_m(float lo, float hi) {
    return __builtin_amdgcn_perm(f2u(hi), f2u(lo), 0x07060302u);
}

__constant__ float c_nf4_big[16] = XFTHIP_NF4_CODE_VALUES;

__device__ inline float silu_big(float x) {
    return x / (1.0f + fast_exp(-x));
}

// MFMA shape: v_mfma_f32_32x32x16_bf16 with the activations as the "A" operand (rows = tokens)
// and the widened weights as "B" (columns = output columns), so a lane's accumulators are
// D[m = 8 (j/4) + 4 h + j%4][n = lane & 31] (h = lane >> 5): consecutive lanes hold consecutive
// output columns and the epilogue stores 64-byte row segments.
//
// KIND: weight kind; WN: 32-column tiles per wave (4 waves per block split the columns);
// WM: 32-row activation tiles per block (shared by the waves through LDS); NEED_SUM: accumulate
// row sums of A for the zero-point term; KTAIL: K is not a whole number of tiles.
template <int KIND>
struct StepTraits;
template <>
struct StepTraits<XFTHIP_W_INT8> {
    // a lane of half h takes the whole 16-byte chunks of k groups h and 2 + h (one 128-bit load each):
    // the k index of an MFMA is only a summation index, so lane half h of micro-step (g, sb) stands for
    // k = 32 g + 16 h + 8 sb .. + 7 in both operands
    static constexpr int KTILE = 64, GROUPS = 2, SUB = 2, WREGS = 4, PACKED_K = 64;
};
template <>
struct StepTraits<XFTHIP_W_UINT4> {
    // 16 bytes per lane per k group, 2 MFMAs.  A step covers half a packed tile (two of its four k groups): with the
    // whole 128-deep tile a step the three activation buffers of a 128-row block take 104 KB of LDS, one workgroup a CU
    static constexpr int KTILE = 64, GROUPS = 2, SUB = 2, WREGS = 4, PACKED_K = 128;
};
template <>
struct StepTraits<XFTHIP_W_NF4> {
    static constexpr int KTILE = 64, GROUPS = 2, SUB = 2, WREGS = 4, PACKED_K = 128;
};
template <>
struct StepTraits<XFTHIP_W_BF16> {
    static constexpr int KTILE = 32, GROUPS = 2, SUB = 1, WREGS = 4, PACKED_K = 32;
};

// Row blocks a band: 8, or, with a device-side row count, only as many as the rows the host expects fill: the
// workgroups that do work then come first in the launch order and spread over the CUs; the ones past the count (which
// leave at once) follow them instead of sitting between them.  (Host and device: the grid is sized with it.)
template <int ROWS, bool DEVROWS>
__host__ __device__ inline int band_rows(const SkinnyParams &p) {
    if constexpr (DEVROWS) {
        if (!p.group) {
            const int want = (p.m_hint + ROWS - 1) / ROWS;
            return want < 1 ? 1 : want < 8 ? want : 8;
        }
    }
    return 8;
}

// DEVROWS: the row count (and, for a group of weights, the weight) comes from device memory (SkinnyParams::rows_dev /
// group); a form of its own, so that the plain kernels carry none of it
//
// DIRECT: the activation tiles go from global memory straight into LDS (global_load_lds_dwordx4: a wave instruction
// fills 1 KiB of consecutive LDS, lane after lane, from 64 addresses of its choice) instead of through registers and
// ds_write.  Rows are 128 bytes with no padding; the 16-byte chunk c of row r sits in slot c ^ ((r >> 1) & 7) of its
// row, which a lane gets by choosing the global chunk it fetches, and which keeps the operand reads (32 rows, one
// chunk index) free of bank conflicts.  Four LDS tiles: step k requests tile k + 3, and the barrier that ends a step
// first waits until the wave's requests of the step before are in (vmcnt counts them in order with the weight
// loads).  Without the staging registers the 128 x 256 tile fits two workgroups a CU.  (A deeper form for launches of
// one workgroup a CU - weights four tiles ahead in five register sets, six LDS tiles requested five steps ahead - was
// built and measured no faster, 921 / 919 against 953 / 956 TFLOP/s on 2048 x 4096 x 4096 and 2048 x 4096 x 11008:
// a lone wave a SIMD is not waiting for memory there, it issues its widening and its MFMAs one after the other.)
//
// KG = 2 (DIRECT only): the form for launches of at most one block a CU.  Eight waves a workgroup: waves 0..3 take the
// first half of K, waves 4..7 the second, each group with LDS tiles and a pipeline of its own (the step barriers are
// the workgroup's, both groups take the same number of steps), so that a SIMD has two waves to issue from as it has
// with two blocks a CU.  After the k loop the second group hands its accumulators (and row sums) to the first
// through LDS, which runs the epilogue.
template <int KIND, int WN, int WM, bool NEED_SUM, bool KTAIL, bool DEVROWS = false, bool DIRECT = false, int WSETS = 3, int KG = 1>
__global__ __launch_bounds__(256 * KG, (DIRECT && KG == 1) ? 2 : 1) void qgemm_mfma_kernel(SkinnyParams p, int nblocks_n, int nblocks_m) {
    using T = StepTraits<KIND>;
    constexpr int KTILE = T::KTILE, GROUPS = T::GROUPS, SUB = T::SUB, WREGS = T::WREGS;
    constexpr int PACKED_K = T::PACKED_K, STEPS_PER_TILE = PACKED_K / KTILE; // k of a packed 1-KiB tile; steps that share one
    constexpr int ROWS = 32 * WM;
    constexpr int ROWB = DIRECT ? KTILE * 2 : KTILE * 2 + 16; // LDS row pitch in bytes (padded when staged through registers)
    static_assert(!DIRECT || (KTILE == 64 && !KTAIL && !DEVROWS && ROWS % 32 == 0), "direct-to-LDS form: 64-deep steps, whole k tiles, host-side row count");
    constexpr int CHUNKS_PER_ROW = KTILE / 8; // 16-byte chunks
    constexpr int TOTAL_CHUNKS = ROWS * CHUNKS_PER_ROW;
    constexpr int ALOADS = TOTAL_CHUNKS / 256;
    static_assert(TOTAL_CHUNKS % 256 == 0, "activation tile must split evenly over the block");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    static_assert(KG == 1 || (KG == 2 && DIRECT), "K groups: the direct-to-LDS form only");
    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3; // wave: position among the 4 waves that split the columns
    const int kgroup = KG == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;
    const int h = lane >> 5, nl = lane & 31;
    const int part_rows = p.M; // rows of a K part: the host's bound, also when the device knows fewer
    // workgroup -> (K part, column block, row block).  Row blocks are walked in bands of 8; a unit of work is one
    // (band, K part, column block): its 8 workgroups share the column block's weights.  Workgroup ids go round the 8
    // XCDs in launch order, so the units are dealt out to the XCDs one by one - an XCD runs the 8 workgroups of a unit
    // next to each other (the weights pass through its L2 once) and its units follow each other column block by column
    // block inside a band (the band's activation rows stay in its L2 while the weights stream past them) - and the
    // XCDs carry the same load whatever the number of column blocks (43 blocks of 256 columns dealt out block by block
    // would give three XCDs 6 and five XCDs 5).
    int nb, mb, part;
    {
        const int BAND = band_rows<ROWS, DEVROWS>(p);
        const int parts = p.ksplit > 1 ? p.ksplit : 1;
        const int id = blockIdx.x, xcd = id & 7, slot = id >> 3; // gridDim.x is a multiple of 8
        const int nbands = (nblocks_m + BAND - 1) / BAND;
        const int units = nbands * parts * nblocks_n;
        const int unit = (slot / BAND) * 8 + xcd;
        if (unit >= units) return;
        const int band = unit / (parts * nblocks_n), rem = unit - band * (parts * nblocks_n);
        part = rem / nblocks_n;
        nb = rem - part * nblocks_n;
        mb = band * BAND + slot % BAND;
        if (mb >= nblocks_m) return;
    }
    int c_row = 0, part_row = 0; // first row of this GEMM in C and in a K part
    if constexpr (DEVROWS) {
    if (p.group) {
        // several weights of one shape behind one launch: the row blocks of all of them are numbered in a
        // row, weight after weight, by their device-side row counts; blocks past the last one leave
        int e = 0, first = 0;
        for (; e < p.group_n; ++e) {
            const int nblk = (p.rows_dev[e * p.rows_stride] + ROWS - 1) / ROWS;
            if (mb < first + nblk) break;
            first += nblk;
        }
        if (e == p.group_n) return;
        mb -= first;
        const int *rec = p.rows_dev + e * p.rows_stride;
        p.M = rec[0];
        p.A += (size_t)rec[1] * p.lda;
        c_row = part_row = rec[2];
        p.packed = p.group[e].packed;
        p.scale = p.group[e].scale;
        p.zero = p.group[e].zero;
    } else if (p.rows_dev) {
        p.M = p.rows_dev[0] < part_rows ? p.rows_dev[0] : part_rows;
        p.A += (size_t)p.rows_dev[1] * p.lda;
        c_row = p.rows_dev[2]; // the K parts hold local rows, the kernel that adds them shifts
    }
    p.C = (char *)p.C + (size_t)c_row * p.ldc * (p.c_dtype == XFTHIP_F32 ? 4 : 2);
    }
    if (p.ksplit > 1) {
        // this workgroup owns a range of k tiles: shift the operands to it, the result goes to its part
        const int kt0 = part * p.split_ktiles;
        const int k_left = p.K - kt0 * PACKED_K, k_span = p.split_ktiles * PACKED_K; // (split_ktiles counts packed tiles)
        p.packed += (size_t)kt0 * 1024;
        p.A += (size_t)kt0 * PACKED_K;
        p.K = k_left < k_span ? k_left : k_span;
        p.C = p.split_part + ((size_t)part * part_rows + part_row) * p.N;
        p.ldc = p.N;
        p.c_dtype = XFTHIP_F32;
        p.epi = XFTHIP_EPI_NONE;
    }
    if constexpr (KG == 2) {
        // (the launcher takes this form only for a K of a whole number of packed tiles per group)
        const int half_k = p.K / 2;
        p.packed += (size_t)kgroup * (half_k / PACKED_K) * 1024;
        p.A += (size_t)kgroup * half_k;
        p.K = half_k;
    }
    const int n32_0 = (nb * 4 + wave) * WN; // first 32-column tile of this wave
    const int m0 = mb * ROWS;
    if constexpr (DEVROWS) {
        if (m0 >= p.M) return; // fewer rows than the grid was sized for (the whole workgroup leaves)
    }

    uint2 *lut = nullptr;
    unsigned char *abuf_base = lds;
    if constexpr (KIND == XFTHIP_W_NF4) {
        // DIRECT: the table sits behind the tiles, which then start at LDS offset 0 of the workgroup and end below 64 KiB
        // (the requests carry their LDS address in M0)
        lut = (uint2 *)(DIRECT ? lds + KG * 4 * ROWS * ROWB + (KG == 2 ? 1024 : 0) : lds);
        abuf_base = DIRECT ? lds : lds + 2048;
        if (threadIdx.x < 256) {
            const int i = threadIdx.x;
            const float c0 = c_nf4_big[i & 15], c1 = c_nf4_big[i >> 4];
            const uint32_t h0 = f32_to_bf16_ref(c0), h1 = f32_to_bf16_ref(c1);
            const uint32_t l0 = f32_to_bf16_ref(c0 - bf16_to_f32((uint16_t)h0));
            const uint32_t l1 = f32_to_bf16_ref(c1 - bf16_to_f32((uint16_t)h1));
            lut[i] = make_uint2(h0 | (h1 << 16), l0 | (l1 << 16));
        }
    }

    if constexpr (KG == 2) abuf_base += kgroup * (4 * ROWS * ROWB); // this group's LDS tiles
    f32x16 acc[WN][WM];
    f32x16 accS[WM];
#pragma unroll
    for (int t = 0; t < WN; ++t)
#pragma unroll
        for (int m = 0; m < WM; ++m)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[t][m][j] = 0.0f;
#pragma unroll
    for (int m = 0; m < WM; ++m)
#pragma unroll
        for (int j = 0; j < 16; ++j) accS[m][j] = 0.0f;

    // weight source of this lane: 16-column packed tile (2 per 32-column MFMA tile), chunk of
    // its column inside the tile, and which 8-byte half (INT8) / dword pair (4-bit) it uses
    const uint8_t *wbase[WN];
#pragma unroll
    for (int t = 0; t < WN; ++t) {
        int nt = (n32_0 + t) * 2 + (nl >> 4);
        nt = nt < p.NTILES ? nt : p.NTILES - 1;
        wbase[t] = p.packed + (size_t)nt * p.KT * 1024 + (nl & 15) * 16;
    }
    constexpr int ROW_STEP = 256 / CHUNKS_PER_ROW;
    const int a_kc = threadIdx.x % CHUNKS_PER_ROW;
    const int a_row0 = threadIdx.x / CHUNKS_PER_ROW;
    uint32_t a_off[ALOADS];
#pragma unroll
    for (int i = 0; i < ALOADS; ++i) {
        if constexpr (DIRECT) {
            // request i of this wave fills LDS chunks 64 (ALOADS wave + i) ..+ 63 = rows 8 (ALOADS wave + i) ..+ 7;
            // this lane's chunk is slot lane & 7 of row lane >> 3 of those, which holds global chunk slot ^ swizzle(row)
            const int r = 8 * (ALOADS * wave + i) + (lane >> 3);
            int row = m0 + r;
            row = row < p.M ? row : p.M - 1;
            a_off[i] = ((uint32_t)row * (uint32_t)p.lda + ((lane & 7) ^ ((r >> 1) & 7)) * 8) * 2; // in bytes
        } else {
            int row = m0 + a_row0 + i * ROW_STEP;
            row = row < p.M ? row : p.M - 1;
            a_off[i] = (uint32_t)row * (uint32_t)p.lda + a_kc * 8;
        }
    }

    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    // Three-stage pipeline over k tiles.  At the start of step k: LDS buffers k % 3 and (k + 1) % 3 hold the
    // activation tiles k and k + 1 (published by earlier barriers), the weight registers of sets k % WSETS
    // .. (k + WSETS - 2) % WSETS hold or await tiles k .. k + WSETS - 2, the activation registers await tile k + 2,
    // and the first MFMA operands of tile k are already in registers.  Step k sends the loads of weight
    // tile k + WSETS - 1 and activation tile k + 4, moves activation tile k + 2 from registers into LDS buffer
    // (k + 2) % 3 (last read two steps ago), computes tile k while reading each next operand set a
    // micro-step ahead (the last one from tile k + 1's buffer), and ends in the barrier that publishes
    // buffer (k + 2) % 3.  Every wait is for loads at least one full step old, and the MFMAs after a
    // barrier never wait for an LDS read.
    constexpr int MICRO = GROUPS * SUB;
    // weight register sets: tile j in set j % WSETS, loaded WSETS - 1 steps ahead.  Three for the large tiles (MFMA
    // bound; the registers are the accumulators'); six for the 32- and 64-row tiles, whose launches are bound by
    // the weights' trip from HBM - with two tiles in flight a step of such a workgroup waited most of a round trip
    static_assert(WSETS % 3 == 0 && (!DIRECT || WSETS == 3), "the activation side of the pipeline walks three buffers");
    constexpr int WD = WSETS - 1;
    uint32_t wreg[WSETS][GROUPS][WN][WREGS];
    u32x4 areg[3][ALOADS];
    const int kt_n = (p.K + KTILE - 1) / KTILE;

    // weight codes of k group gq of tile kt_ into register set buf
    auto load_w_part = [&](int buf, int kt_, int gq) {
        const int kt = kt_ < kt_n ? kt_ : kt_n - 1; // past the end: a valid tile, never used
#pragma unroll
        for (int t = 0; t < WN; ++t) {
            if constexpr (KIND == XFTHIP_W_INT8) {
                const u32x4 v = *(const u32x4 *)(wbase[t] + (size_t)kt * 1024 + (2 * gq + h) * 256);
                wreg[buf][gq][t][0] = v[0]; wreg[buf][gq][t][1] = v[1]; wreg[buf][gq][t][2] = v[2]; wreg[buf][gq][t][3] = v[3];
            } else if constexpr (KIND == XFTHIP_W_BF16) {
                // chunk g = 2 s + h holds k = 8 g .. 8 g + 7
                const u32x4 v = *(const u32x4 *)(wbase[t] + (size_t)kt * 1024 + (2 * gq + h) * 256);
                wreg[buf][gq][t][0] = v[0]; wreg[buf][gq][t][1] = v[1]; wreg[buf][gq][t][2] = v[2]; wreg[buf][gq][t][3] = v[3];
            } else {
                const u32x4 v = *(const u32x4 *)(wbase[t] + (size_t)(kt / STEPS_PER_TILE) * 1024 + ((kt % STEPS_PER_TILE) * GROUPS + gq) * 256);
                wreg[buf][gq][t][0] = v[0]; wreg[buf][gq][t][1] = v[1]; wreg[buf][gq][t][2] = v[2]; wreg[buf][gq][t][3] = v[3];
            }
        }
    };
    auto load_w = [&](int buf, int kt_) {
#pragma unroll
        for (int gq = 0; gq < GROUPS; ++gq) load_w_part(buf, kt_, gq);
    };
    // 16-byte chunk i of this thread's share of activation tile kt_ into register set `set`
    auto load_a_part = [&](int set, int kt_, int i) {
        const int kt = kt_ < kt_n ? kt_ : kt_n - 1;
        if constexpr (KTAIL) {
            const int k = kt * KTILE + a_kc * 8;
            const bool v = k < p.K;
            const u32x4 a = *(const u32x4 *)(p.A + a_off[i] + (v ? (size_t)kt * KTILE : (size_t)0) - (v ? 0 : a_kc * 8));
            areg[set][i] = v ? a : zero4;
        } else {
            areg[set][i] = *(const u32x4 *)(p.A + a_off[i] + (size_t)kt * KTILE);
        }
    };
    auto load_a = [&](int set, int kt_) {
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) load_a_part(set, kt_, i);
    };
    // DIRECT: request i of this wave's share of activation tile kt_ into LDS tile buf (wave-uniform)
    // (Written as assembly: after the compiler's own builtin for this instruction it makes every later wait for a load
    // or an LDS read a wait for all of them - an instruction of the flat family that touches both memories - which
    // takes the two-tiles-ahead weight loads out of flight at every step.  Unaware of these requests, the compiler's
    // counted waits for the weight loads come out a few requests early, never late: the counter retires in order.
    // M0 carries the LDS address of the wave's first lane; one wait state between writing it and the request.  The
    // compiler holds nothing in M0 across statements - it is a reserved register that it writes right in front of each
    // instruction of its own that reads it - so the statement may overwrite it.)
    const uint32_t lds_tiles = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)abuf_base +
            ALOADS * 1024 * (uint32_t)__builtin_amdgcn_readfirstlane(wave);
    const uint64_t a_bits = (uint64_t)(uintptr_t)p.A; // the same in every lane; said so, for a scalar register pair
    const uint16_t *a_uniform = (const uint16_t *)(uintptr_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(a_bits >> 32)) << 32) |
            (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a_bits));
    auto direct_a_part = [&](int buf, int kt_, int i) {
        const int kt = __builtin_amdgcn_readfirstlane(kt_ < kt_n ? kt_ : kt_n - 1);
        const uint32_t dst = lds_tiles + buf * (ROWS * ROWB) + i * 1024;
        const uint16_t *src = a_uniform + (size_t)kt * KTILE;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(a_off[i]), "s"(src) : "memory");
    };
    auto direct_a = [&](int buf, int kt_) {
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) direct_a_part(buf, kt_, i);
    };
    // NEED_SUM: the row sums of A (zero-point term) are gathered where the rows are staged: the thread that moves a
    // 16-byte chunk into LDS adds its 8 values to a partial of its own; the partials of a row's chunks are joined after
    // the k loop.  (They used to come from one more MFMA a row tile and micro-step against a tile of ones: as many
    // MFMAs again as the product itself with one column tile a wave, and 16 WM accumulator registers.)
    float rs_part[ALOADS];
#pragma unroll
    for (int i = 0; i < ALOADS; ++i) rs_part[i] = 0.0f;
    auto store_a_part = [&](int set, int buf, int i, bool real_tile) {
        unsigned char *dst = abuf_base + buf * (ROWS * ROWB);
        *(u32x4 *)(dst + (a_row0 + i * ROW_STEP) * ROWB + a_kc * 16) = areg[set][i];
        if constexpr (NEED_SUM) {
            if (real_tile) { // (uniform: tiles past the end of K are copies of the last one)
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t u = areg[set][i][w];
                    rs_part[i] += u2f(u << 16) + u2f(u & 0xFFFF0000u);
                }
            }
        }
    };
    auto store_a = [&](int set, int buf, bool real_tile) {
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) store_a_part(set, buf, i, real_tile);
    };
    // k offset (elements) of micro-step ms inside a tile: lane (row/col, h) holds k = koff .. koff + 7
    auto koff_of = [&](int ms) {
        const int gq = ms / SUB, sb = ms % SUB;
        return KIND == XFTHIP_W_INT8 ? 32 * gq + 16 * h + 8 * sb : KIND == XFTHIP_W_BF16 ? 16 * gq + 8 * h : 32 * gq + 16 * sb + 8 * h;
    };
    // DIRECT + NEED_SUM: wave w walks the row tiles in the order w, w + 1, .. (mod WM), so that the operand it sums for
    // the zero-point term (below) is always the first one it reads - no branch on the wave number inside the k loop
    constexpr bool ROTATE = DIRECT && NEED_SUM;
    const int wave_first = ROTATE ? __builtin_amdgcn_readfirstlane(wave) : 0;
    auto row_tile = [&](int m) { return ROTATE ? (m + wave_first) % WM : m; };
    MFrag afr[2][WM];
    auto read_frags = [&](int slot, int ab, int ms) {
        const unsigned char *src = abuf_base + ab * (ROWS * ROWB) + nl * ROWB +
                (DIRECT ? (((koff_of(ms) >> 3) ^ ((nl >> 1) & 7)) << 4) : koff_of(ms) * 2);
#pragma unroll
        for (int m = 0; m < WM; ++m) afr[slot][m].q = *(const u32x4 *)(src + row_tile(m) * 32 * ROWB);
    };
    // one MFMA k step = 16 k.  Operands of micro-step ms sit in afr[ms & 1]; the next set (of the
    // next tile's buffer after the last micro-step) is read while this one's MFMAs run.
    // Besides the MFMAs of tile kt (weight set w_cur, LDS buffer lds_cur), a step sends the loads of weight
    // tile kt + WD (into set w_load) and activation tile kt + 4 (into register set a_load) and moves
    // activation tile kt + 2 (register set a_stage, loaded two steps ago) into LDS buffer
    // a_stage: one slice of each per micro-step, so that no wave ever queues a burst of memory
    // instructions in front of its MFMAs (a wave issues in order; 4 waves sending 12 loads each right
    // after a barrier kept the MFMA pipes waiting for the address path).
    constexpr int A_EVERY = MICRO / ALOADS;
    static_assert(MICRO % ALOADS == 0, "activation slices must spread evenly over the micro-steps");
    // widened MFMA operands of (weight set wb, micro-step ms, column tile t)
    auto widen = [&](int wb, int ms, int t, MFrag &whi, MFrag &wlo) {
        const int gq = ms / SUB, sb = ms % SUB;
        if constexpr (KIND == XFTHIP_W_INT8) {
            const uint32_t x = wreg[wb][gq][t][2 * sb], y = wreg[wb][gq][t][2 * sb + 1];
            whi.u[0] = pack_hi16_m((float)(int)(int8_t)(x), (float)(int)(int8_t)(x >> 8));
            whi.u[1] = pack_hi16_m((float)(int)(int8_t)(x >> 16), (float)((int)x >> 24));
            whi.u[2] = pack_hi16_m((float)(int)(int8_t)(y), (float)(int)(int8_t)(y >> 8));
            whi.u[3] = pack_hi16_m((float)(int)(int8_t)(y >> 16), (float)((int)y >> 24));
        } else if constexpr (KIND == XFTHIP_W_BF16) {
            whi.u[0] = wreg[wb][gq][t][0]; whi.u[1] = wreg[wb][gq][t][1];
            whi.u[2] = wreg[wb][gq][t][2]; whi.u[3] = wreg[wb][gq][t][3];
        } else {
            // codes 16 sb + 8 h .. + 8 of the lane's 32-code chunk = dword 2 sb + h
            const uint32_t x0 = wreg[wb][gq][t][2 * sb], x1 = wreg[wb][gq][t][2 * sb + 1];
            const uint32_t x = h ? x1 : x0;
            if constexpr (KIND == XFTHIP_W_UINT4) {
                whi.u[0] = (x & 0x000F000Fu) | 0x43004300u;
                whi.u[1] = ((x >> 4) & 0x000F000Fu) | 0x43004300u;
                whi.u[2] = ((x >> 8) & 0x000F000Fu) | 0x43004300u;
                whi.u[3] = ((x >> 12) & 0x000F000Fu) | 0x43004300u;
            } else {
                const uint2 e0 = lut[x & 0xFF], e1 = lut[(x >> 8) & 0xFF], e2 = lut[(x >> 16) & 0xFF], e3 = lut[x >> 24];
                whi.u[0] = e0.x; whi.u[1] = e1.x; whi.u[2] = e2.x; whi.u[3] = e3.x;
                wlo.u[0] = e0.y; wlo.u[1] = e1.y; wlo.u[2] = e2.y; wlo.u[3] = e3.y;
            }
        }
    };
    // The operands of slot (ms, t) are widened while the MFMAs of the slot before run: wcur_* enter
    // a step holding slot (0, 0) of its tile and leave it holding slot (0, 0) of the next tile.
    MFrag wcur_hi, wcur_lo;
    // the explicit interleave below pays for the BF16 kind (no widening work to hide: +5 %) and costs
    // the INT8 kind 6 % on 128 x 128 tiles, where the compiler's own order is better
    constexpr bool SGB = KIND == XFTHIP_W_BF16;
    // VALU instructions one widening takes (a hint for the instruction interleave below)
    constexpr int VW = KIND == XFTHIP_W_INT8 ? 12 : KIND == XFTHIP_W_UINT4 ? 9 : KIND == XFTHIP_W_NF4 ? 6 : 0;
    constexpr int VPER = (VW + WM - 1) / WM;
    // w_cur / w_next / w_load: weight register sets of tiles kt_cur, kt_cur + 1 and kt_cur + WD (the one this step loads).
    // lds_cur / lds_next: LDS tiles of activation tiles kt_cur and kt_cur + 1.  DIRECT: lds_req, the LDS tile this step
    // requests activation tile kt_cur + 3 into; staged form: a_load, the register set tile kt_cur + 4 is loaded into,
    // and a_stage, the register set (and LDS tile of the same number) tile kt_cur + 2 moves from (to)
    float rs_direct = 0.0f; // DIRECT + NEED_SUM: wave w sums the rows of row tile w, the first operand it reads
    auto compute = [&](int w_cur, int w_next, int w_load, int a_load, int a_stage, int kt_cur, int lds_cur, int lds_next, int lds_req) {
#pragma unroll
        for (int ms = 0; ms < MICRO; ++ms) {
            const int gq = ms / SUB, sb = ms % SUB;
            if (sb == 0) load_w_part(w_load, kt_cur + WD, gq);
            if (ms % A_EVERY == 0) {
                if constexpr (DIRECT) {
                    direct_a_part(lds_req, kt_cur + 3, ms / A_EVERY);
                } else {
                    load_a_part(a_load, kt_cur + 4, ms / A_EVERY);
                    store_a_part(a_stage, a_stage, ms / A_EVERY, kt_cur + 2 < kt_n);
                }
            }
            if (ms + 1 < MICRO)
                read_frags((ms + 1) & 1, lds_cur, ms + 1);
            else
                read_frags((ms + 1) & 1, lds_next, 0);
            const MFrag *a = afr[ms & 1];
            if constexpr (DIRECT && NEED_SUM) {
                static_assert(!(DIRECT && NEED_SUM) || WM == 4, "one row tile a wave");
                typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
                const bf16x2_t ones2 = __builtin_bit_cast(bf16x2_t, 0x3F803F80u);
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    rs_direct = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a[0].u[w]), ones2, rs_direct, false);
            }
#pragma unroll
            for (int t = 0; t < WN; ++t) {
                MFrag nhi, nlo;
                if (t + 1 < WN)
                    widen(w_cur, ms, t + 1, nhi, nlo);
                else if (ms + 1 < MICRO)
                    widen(w_cur, ms + 1, 0, nhi, nlo);
                else
                    widen(w_next, 0, 0, nhi, nlo); // the next tile's set: loaded in an earlier step
#pragma unroll
                for (int m = 0; m < WM; ++m) {
                    if constexpr (KIND == XFTHIP_W_NF4)
                        acc[t][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m].v, wcur_lo.v, acc[t][m], 0, 0, 0);
                    acc[t][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m].v, wcur_hi.v, acc[t][m], 0, 0, 0);
                }
                wcur_hi = nhi;
                if constexpr (KIND == XFTHIP_W_NF4) wcur_lo = nlo;
                if constexpr (SGB) {
                    // order of the slot's instructions: its memory instructions first, then one MFMA at a
                    // time with a share of the widening and (first column tile) one LDS read behind it
                    if (t == 0) {
                        if (sb == 0) {
#pragma unroll
                            for (int tt = 0; tt < WN; ++tt) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        }
                        if (ms % A_EVERY == 0) {
                            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                        }
                    }
#pragma unroll
                    for (int m = 0; m < WM; ++m) {
                        __builtin_amdgcn_sched_group_barrier(0x008, KIND == XFTHIP_W_NF4 ? 2 : 1, 0);
                        if (t == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        if (VPER > 0) __builtin_amdgcn_sched_group_barrier(0x002, VPER, 0);
                    }
                }
            }
        }
    };

#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
    // memory requests a wave sends per step (weight loads + activation requests), in program order
    constexpr int REQS_PER_STEP = GROUPS * WN + ALOADS;
    int kt = 0;
    if constexpr (DIRECT) {
        // prologue: activation tiles 0, 1 and 2 in LDS, weight tiles 0 and 1 under way
        load_w(0, 0);
        direct_a(0, 0);
        load_w(1, 1);
        direct_a(1, 1);
        direct_a(2, 2);
        XFT_FENCE();
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    } else {
    // prologue: tiles 0 and 1 in LDS, weight tiles 0 and 1 and activation tiles 2 and 3 under way
    load_w(0, 0);
    load_a(0, 0);
    load_w(1, 1);
    load_a(1, 1);
    load_a(2, 2);
#pragma unroll
    for (int i = 2; i < WD; ++i) load_w(i, i);
    XFT_FENCE();
    store_a(0, 0, true);
    XFT_FENCE();
    load_a(0, 3);
    XFT_FENCE();
    store_a(1, 1, kt_n > 1);
    __syncthreads();
    }
    read_frags(0, 0, 0);
    widen(0, 0, 0, wcur_hi, wcur_lo);
    // step k with s = k % 3 (static): tile j lives in weight set, activation register set and LDS buffer j % 3
    // (DIRECT: LDS tile j % 4; the barrier first waits for this wave's requests of the step before - everything but the
    // REQS_PER_STEP youngest - and for its LDS reads, so the tile published is complete and the tile freed is read)
#define XFT_STEP(s)                                        \
    {                                                      \
        if constexpr (DIRECT) {                            \
            compute((s), ((s) + 1) % 3, ((s) + 2) % 3, 0, 0, kt, kt & 3, (kt + 1) & 3, (kt + 3) & 3); \
            XFT_FENCE();                                   \
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(REQS_PER_STEP) : "memory"); \
        } else {                                           \
            compute((s), ((s) + 1) % WSETS, ((s) + WD) % WSETS, ((s) + 1) % 3, ((s) + 2) % 3, kt, (s) % 3, ((s) + 1) % 3, 0); \
            XFT_FENCE();                                   \
            __syncthreads();                               \
        }                                                  \
        ++kt;                                              \
    }
    if constexpr (WSETS == 6) {
        while (kt + 6 <= kt_n) {
            XFT_STEP(0) XFT_STEP(1) XFT_STEP(2) XFT_STEP(3) XFT_STEP(4) XFT_STEP(5)
        }
        if (kt < kt_n) XFT_STEP(0)
        if (kt < kt_n) XFT_STEP(1)
        if (kt < kt_n) XFT_STEP(2)
        if (kt < kt_n) XFT_STEP(3)
        if (kt < kt_n) XFT_STEP(4)
    } else {
        while (kt + 3 <= kt_n) {
            XFT_STEP(0) XFT_STEP(1) XFT_STEP(2)
        }
        if (kt < kt_n) XFT_STEP(0)
        if (kt < kt_n) XFT_STEP(1)
    }
#undef XFT_STEP
#undef XFT_FENCE

    // ---- epilogue: lane holds C[m0 + 32 mt + 8 (j/4) + 4 h + j%4][32 (n32_0 + t) + nl] ----
    // A lane owns 16 rows of ONE column.  Finishing and storing every element from the accumulator
    // registers costs a 64-bit index, bounds tests and a type conversion in 128 unrolled copies a
    // lane, which made the epilogue of a 2048 x 4096 result take 23 us (the k loop of K = 4096: 75).
    // Instead each wave drops one 32-row block of scaled results at a time, as fp32, into an LDS
    // patch of its own (one ds_write with a constant offset per element), then walks the patch in
    // 8-column chunks, consecutive lanes along a row: residual, conversion and 16-byte stores run
    // in that short loop.
    constexpr int OPITCH = 32 * WN * 4 + 32; // patch row pitch in bytes
    if constexpr (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the requests past the last tile have landed
    __syncthreads(); // every wave is past its last read of the activation tiles
    if constexpr (KG == 2) {
        // the second K group hands its accumulators over, [wave][register][lane] floats from the start of LDS (exactly
        // the two groups' tiles), its row sums behind them
        float *hand = (float *)lds + (size_t)wave * (WN * WM * 16) * 64 + lane;
        float *hand_rs = (float *)(lds + 2 * 4 * ROWS * ROWB) + wave * 64 + lane;
        if (kgroup == 1) {
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int m = 0; m < WM; ++m)
#pragma unroll
                    for (int j = 0; j < 16; ++j) hand[((t * WM + m) * 16 + j) * 64] = acc[t][m][j];
            if constexpr (NEED_SUM) *hand_rs = rs_direct;
        }
        __syncthreads();
        if (kgroup == 0) {
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int m = 0; m < WM; ++m)
#pragma unroll
                    for (int j = 0; j < 16; ++j) acc[t][m][j] += hand[((t * WM + m) * 16 + j) * 64];
            if constexpr (NEED_SUM) rs_direct += *hand_rs;
        }
        __syncthreads(); // (the result patches below overwrite what was handed over)
        abuf_base = lds;
    }
    unsigned char *obuf = abuf_base + wave * (32 * OPITCH);
    if constexpr (NEED_SUM) {
        // join the partial sums of a row's chunks (adjacent lanes), hand them over through LDS behind the patches, and
        // give every lane the sums of the 16 rows it holds results of
        float *rowsum = (float *)(abuf_base + 4 * 32 * OPITCH);
        if constexpr (DIRECT) {
            // lane halves hold the two halves of a row's k range
            const float v = rs_direct + __shfl_xor(rs_direct, 32, 64);
            if (h == 0 && kgroup == 0) rowsum[32 * wave + nl] = v;
        } else {
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) {
            float v = rs_part[i];
#pragma unroll
            for (int off = 1; off < CHUNKS_PER_ROW; off <<= 1) v += __shfl_xor(v, off, 64);
            if (a_kc == 0) rowsum[a_row0 + i * ROW_STEP] = v;
        }
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < WM; ++m)
#pragma unroll
            for (int j = 0; j < 16; ++j) accS[m][j] = rowsum[32 * row_tile(m) + 8 * (j >> 2) + 4 * h + (j & 3)];
    }
    if (KG == 2 && kgroup == 1) return; // (no workgroup barrier from here on)
    const bool c_wide = (((size_t)p.C | ((size_t)p.ldc * (p.c_dtype == XFTHIP_F32 ? 4 : 2))) & 15) == 0;
    const bool res_wide = (((size_t)p.res | ((size_t)p.ldres * (p.res_dtype == XFTHIP_F32 ? 4 : 2))) & 15) == 0;
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    auto put_at = [&](float *base, int t_cols, int j, float x) { base[(8 * (j >> 2) + (j & 3)) * (OPITCH / 4) + t_cols] = x; };
    // rows [32 m, 32 m + 32) of the patch, strip_cols wide, go to output columns col0 .. col_end - 1
    auto flush = [&](auto epi_tag, int m, int col0, int strip_cols, int col_end) {
        constexpr int EPI = decltype(epi_tag)::value;
        constexpr bool HAS_RES = EPI == XFTHIP_EPI_RESMUL || EPI == XFTHIP_EPI_RESIDENTIAL || EPI == XFTHIP_EPI_RESEXT;
        wave_sync();
        const int cpr = strip_cols >> 3; // 8-column chunks a row: 2, 4 or 8
        const int cpr_log2 = __builtin_ctz(cpr);
        for (int idx = lane; idx < 32 * cpr; idx += 64) {
            const int r = idx >> cpr_log2, ch = idx & (cpr - 1);
            const int row = m0 + 32 * m + r;
            const int c = col0 + 8 * ch;
            if (row >= p.M || c >= col_end) continue;
            const float *src = (const float *)(obuf + r * OPITCH) + 8 * ch;
            const f32x4 lo = *(const f32x4 *)src, hi = *(const f32x4 *)(src + 4);
            float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const bool full = c + 8 <= col_end;
            if constexpr (HAS_RES) {
                const size_t ri = (size_t)row * p.ldres + c;
                float rv[8];
                if (full && res_wide) {
                    if (p.res_dtype == XFTHIP_F32) {
                        const f32x4 r0 = *(const f32x4 *)((const float *)p.res + ri), r1 = *(const f32x4 *)((const float *)p.res + ri + 4);
                        rv[0] = r0[0], rv[1] = r0[1], rv[2] = r0[2], rv[3] = r0[3], rv[4] = r1[0], rv[5] = r1[1], rv[6] = r1[2], rv[7] = r1[3];
                    } else {
                        const u32x4 rr = *(const u32x4 *)((const uint16_t *)p.res + ri);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint16_t b0 = (uint16_t)rr[e], b1 = (uint16_t)(rr[e] >> 16);
                            rv[2 * e] = p.res_dtype == XFTHIP_BF16 ? bf16_to_f32(b0) : fp16_bits_to_f32(b0);
                            rv[2 * e + 1] = p.res_dtype == XFTHIP_BF16 ? bf16_to_f32(b1) : fp16_bits_to_f32(b1);
                        }
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) rv[e] = c + e < col_end ? load_as_f32(p.res, p.res_dtype, ri + e) : 0.0f;
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if constexpr (EPI == XFTHIP_EPI_RESMUL) v[e] *= rv[e];
                    if constexpr (EPI == XFTHIP_EPI_RESIDENTIAL) v[e] = v[e] + rv[e];
                    if constexpr (EPI == XFTHIP_EPI_RESEXT) v[e] = fmaf(p.gamma, rv[e], v[e]);
                }
            }
            const size_t ci = (size_t)row * p.ldc + c;
            if (full && c_wide) {
                if (p.c_dtype == XFTHIP_F32) {
                    const f32x4 o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
                    *(f32x4 *)((float *)p.C + ci) = o0;
                    *(f32x4 *)((float *)p.C + ci + 4) = o1;
                } else {
                    u32x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t b0 = p.c_dtype == XFTHIP_BF16 ? f32_to_bf16_sel(v[2 * e]) : f32_to_fp16_bits(v[2 * e]);
                        const uint32_t b1 = p.c_dtype == XFTHIP_BF16 ? f32_to_bf16_sel(v[2 * e + 1]) : f32_to_fp16_bits(v[2 * e + 1]);
                        o[e] = b0 | (b1 << 16);
                    }
                    *(u32x4 *)((uint16_t *)p.C + ci) = o;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (c + e < col_end) store_from_f32(p.C, p.c_dtype, ci + e, v[e]);
            }
        }
        wave_sync();
    };
    auto run_epilogue = [&](auto epi_tag) {
        constexpr int EPI = decltype(epi_tag)::value;
        float s[WN], z[WN], bv[WN];
#pragma unroll
        for (int t = 0; t < WN; ++t) {
            const int np = (n32_0 + t) * 32 + nl;
            s[t] = 1.0f, z[t] = 0.0f, bv[t] = 0.0f;
            if constexpr (KIND != XFTHIP_W_BF16) s[t] = p.scale[np < p.NTILES * 16 ? np : 0];
            if constexpr (KIND == XFTHIP_W_UINT4 || (KIND == XFTHIP_W_INT8 && NEED_SUM)) z[t] = p.zero ? p.zero[np < p.NTILES * 16 ? np : 0] : 0.0f;
            if constexpr (EPI == XFTHIP_EPI_BIAS || EPI == XFTHIP_EPI_RESIDENTIAL || EPI == XFTHIP_EPI_RESEXT) bv[t] = (p.bias && np < p.N) ? p.bias[np] : 0.0f;
        }
        float *put_base = (float *)(obuf + 4 * h * OPITCH) + nl;
#pragma unroll
        for (int m = 0; m < WM; ++m) {
#pragma unroll
            for (int t = 0; t < WN; ++t) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    float x = acc[t][m][j];
                    if constexpr (KIND == XFTHIP_W_UINT4) {
                        x = fmaf(s[t], x - 128.0f * accS[m][j], z[t] * accS[m][j]);
                    } else if constexpr (KIND == XFTHIP_W_INT8) {
                        x = s[t] * x;
                        if constexpr (NEED_SUM) x = fmaf(z[t], accS[m][j], x);
                    } else if constexpr (KIND == XFTHIP_W_NF4) {
                        x = s[t] * x;
                    }
                    if constexpr (EPI == XFTHIP_EPI_BIAS || EPI == XFTHIP_EPI_RESIDENTIAL || EPI == XFTHIP_EPI_RESEXT) x += bv[t];
                    if constexpr (EPI == XFTHIP_EPI_SILU) x = silu_big(x);
                    if constexpr (EPI == XFTHIP_EPI_GELU) {
                        const float e = fast_exp(1.702f * x);
                        x = e / (e + 1.0f) * x;
                    }
                    put_at(put_base, 32 * t, j, x); // the residual operand joins in flush()
                }
            }
            flush(epi_tag, row_tile(m), n32_0 * 32, 32 * WN, p.N);
        }
    };
    if (p.gateup) {
        // packed columns alternate 16 gate / 16 up: lanes nl < 16 hold gate, nl >= 16 the matching up
        float s[WN], z[WN];
#pragma unroll
        for (int t = 0; t < WN; ++t) {
            const int np = (n32_0 + t) * 32 + nl;
            s[t] = 1.0f, z[t] = 0.0f;
            if constexpr (KIND != XFTHIP_W_BF16) s[t] = p.scale[np < p.NTILES * 16 ? np : 0];
            if constexpr (KIND == XFTHIP_W_UINT4 || (KIND == XFTHIP_W_INT8 && NEED_SUM)) z[t] = p.zero ? p.zero[np < p.NTILES * 16 ? np : 0] : 0.0f;
        }
        // gate lanes write output column 16 t + nl of the strip; the up lanes' copies of the
        // product land in the unused columns behind the strip, which flush() never reads
        float *put_base = (float *)(obuf + 4 * h * OPITCH) + (nl < 16 ? nl : 16 * WN + (nl - 16));
#pragma unroll
        for (int m = 0; m < WM; ++m) {
#pragma unroll
            for (int t = 0; t < WN; ++t) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    float x = acc[t][m][j];
                    if constexpr (KIND == XFTHIP_W_UINT4) {
                        x = fmaf(s[t], x - 128.0f * accS[m][j], z[t] * accS[m][j]);
                    } else if constexpr (KIND == XFTHIP_W_INT8) {
                        x = s[t] * x;
                        if constexpr (NEED_SUM) x = fmaf(z[t], accS[m][j], x);
                    } else if constexpr (KIND == XFTHIP_W_NF4) {
                        x = s[t] * x;
                    }
                    const float other = __shfl_xor(x, 16, 64); // gate <-> up partner
                    put_at(put_base, 16 * t, j, other * silu_big(x));
                }
            }
            flush(std::integral_constant<int, XFTHIP_EPI_NONE> {}, row_tile(m), n32_0 * 16, 16 * WN, p.N / 2);
        }
        return;
    }
    switch (p.epi) {
        case XFTHIP_EPI_BIAS: run_epilogue(std::integral_constant<int, XFTHIP_EPI_BIAS> {}); break;
        case XFTHIP_EPI_SILU: run_epilogue(std::integral_constant<int, XFTHIP_EPI_SILU> {}); break;
        case XFTHIP_EPI_GELU: run_epilogue(std::integral_constant<int, XFTHIP_EPI_GELU> {}); break;
        case XFTHIP_EPI_RESMUL: run_epilogue(std::integral_constant<int, XFTHIP_EPI_RESMUL> {}); break;
        case XFTHIP_EPI_RESIDENTIAL: run_epilogue(std::integral_constant<int, XFTHIP_EPI_RESIDENTIAL> {}); break;
        case XFTHIP_EPI_RESEXT: run_epilogue(std::integral_constant<int, XFTHIP_EPI_RESEXT> {}); break;
        default: run_epilogue(std::integral_constant<int, XFTHIP_EPI_NONE> {}); break;
    }
}

template <int KIND, int WN, int WM, bool NEED_SUM, bool KTAIL, bool DEVROWS = false, bool DIRECT = false, int KG = 1>
static int launch_big2(const SkinnyParams &p, hipStream_t stream) {
    // six weight tiles in flight for the 32- and 64-row tiles (see the kernel), three for the others
    constexpr int WSETS = (!DIRECT && WN == 1 && WM <= 2) ? 6 : 3;
    using T = StepTraits<KIND>;
    constexpr int ROWS = 32 * WM, ROWB = DIRECT ? T::KTILE * 2 : T::KTILE * 2 + 16;
    const int n32 = (p.NTILES + 1) / 2;
    const int nblocks_n = (n32 + 4 * WN - 1) / (4 * WN);
    // a group's row blocks: every weight may end in a partly filled one
    const int nblocks_m = (p.M + ROWS - 1) / ROWS + (p.group ? p.group_n : 0);
    // 8 workgroups a unit of (band of row blocks, K part, column block), the units dealt out to the 8 XCDs
    const int band = band_rows<ROWS, DEVROWS>(p), parts = p.ksplit > 1 ? p.ksplit : 1;
    const long units = (long)((nblocks_m + band - 1) / band) * parts * nblocks_n;
    const long blocks_l = (units + 7) / 8 * 8 * band;
    if (blocks_l > 0x7fffffffL) {
        set_error("qgemm_mfma: too many workgroups");
        return 2;
    }
    const int blocks = (int)blocks_l;
    // the three activation buffers, reused after the k loop by the four waves' output patches
    // (the row sums of the zero-point term sit behind the patches)
    const size_t pipe = (DIRECT ? 4 : 3) * ROWS * ROWB * KG + (KG == 2 ? 1024 : 0), patches = 4 * 32 * (32 * WN * 4 + 32) + (NEED_SUM ? ROWS * sizeof(float) : 0);
    const size_t smem = (pipe > patches ? pipe : patches) + (KIND == XFTHIP_W_NF4 ? 2048 : 0);
    if (smem > 64 * 1024) {
        // more dynamic LDS than the default limit: raise it once per instantiation
        static const hipError_t attr = hipFuncSetAttribute((const void *)qgemm_mfma_kernel<KIND, WN, WM, NEED_SUM, KTAIL, DEVROWS, DIRECT, WSETS, KG>,
                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        XFT_CHECK_HIP(attr);
    }
    hipLaunchKernelGGL((qgemm_mfma_kernel<KIND, WN, WM, NEED_SUM, KTAIL, DEVROWS, DIRECT, WSETS, KG>), dim3(blocks), dim3(256 * KG), smem, stream,
            p, nblocks_n, nblocks_m);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

template <int KIND, int WN, int WM, bool NEED_SUM>
static int launch_big(const SkinnyParams &p, hipStream_t stream) {
    if (p.rows_dev) {
        // device-side row counts: built for the 32- and 64-row tiles only (dispatch_big_tile picks no other then)
        if constexpr (WN == 1 && WM <= 2) {
            if (p.K % StepTraits<KIND>::KTILE != 0) return launch_big2<KIND, WN, WM, NEED_SUM, true, true>(p, stream);
            return launch_big2<KIND, WN, WM, NEED_SUM, false, true>(p, stream);
        } else {
            set_error("qgemm_mfma: no device-side row count for this tile");
            return 2;
        }
    }
    if (p.K % StepTraits<KIND>::KTILE != 0) return launch_big2<KIND, WN, WM, NEED_SUM, true>(p, stream);
    if constexpr (WN == 2 && WM == 4 && KIND != XFTHIP_W_BF16) {
        // whole k tiles: the 128 x 256 tile takes its activations straight into LDS, two workgroups a CU
        // (the kernel keeps a lane's byte offset into the activations in 32 bits)
        if ((size_t)p.M * (size_t)p.lda * 2 < ((size_t)1 << 32)) {
            // at most one block a CU: two K groups a workgroup give every SIMD a second wave (see the kernel)
            const long wgs = (long)(((p.NTILES + 1) / 2 + 4 * WN - 1) / (4 * WN)) * ((p.M + 32 * WM - 1) / (32 * WM));
            // (2048 rows x 4096 columns, K = 4096 / 11008: INT8 963 / 993 against 926 / 934 TFLOP/s on the same box, UINT4
            // 859 / 954 against 812 / 926, NF4 519 / 569 against 492 / 532)
            if (wgs <= device_cu_count() && p.ksplit <= 1 && p.K % (2 * StepTraits<KIND>::PACKED_K) == 0)
                return launch_big2<KIND, WN, WM, NEED_SUM, false, false, true, 2>(p, stream);
            return launch_big2<KIND, WN, WM, NEED_SUM, false, false, true>(p, stream);
        }
    }
    return launch_big2<KIND, WN, WM, NEED_SUM, false>(p, stream);
}

template <int KIND, bool NEED_SUM>
static int dispatch_big_tile(const SkinnyParams &p, hipStream_t stream) {
    const int cus = device_cu_count();
    // Block tile = (4*WN*32 columns) x (WM*32 rows).  The choices below are the measured winners on
    // 4096x{4096,12288,22016} and 11008x4096 weights at 512, 1024 and 2048 rows: 128-row tiles only
    // pay once there are many row blocks to share a weight tile's trip through L2; below that,
    // more and smaller workgroups per CU (whose k loops overlap) win by up to 1.5x.
    const int n32 = (p.NTILES + 1) / 2;
    // the tile is chosen for the rows the host expects; with a device-side row count p.M is only the bound
    const int rows = (p.rows_dev && !p.group && p.m_hint > 0) ? p.m_hint : p.M;
    const long t_large = (long)((n32 + 7) / 8) * ((rows + 127) / 128);
    const long t_mid = (long)((n32 + 3) / 4) * ((rows + 127) / 128);
    const long t_small = (long)((n32 + 3) / 4) * ((rows + 63) / 64);
    if (p.rows_dev) {
        // 32- or 64-row tiles.  A group's weights with more than 32 rows each keep 64-row tiles: the 32-row ones
        // read every weight tile twice, and with all the weights' workgroups side by side there is no CU left to fill.
        if constexpr (KIND != XFTHIP_W_BF16) {
            if (t_small < 2 * cus && !(p.group && p.M > 32 * p.group_n)) return launch_big<KIND, 1, 1, NEED_SUM>(p, stream);
        }
        // (128-row tiles for a group whose weights expect about 64 rows each - one pass over a weight instead of a
        // second row block for the rows past 64 - measured 574 us a sparse MLP layer against 496)
        return launch_big<KIND, 1, 2, NEED_SUM>(p, stream);
    }
    if constexpr (KIND == XFTHIP_W_BF16) {
        if (t_large >= cus) return launch_big<KIND, 2, 4, NEED_SUM>(p, stream);
        if (t_mid >= cus) return launch_big<KIND, 1, 4, NEED_SUM>(p, stream);
        return launch_big<KIND, 1, 2, NEED_SUM>(p, stream);
    } else if constexpr (KIND == XFTHIP_W_INT8) {
        // The 128 x 256 tile with the activations straight into LDS (two workgroups a CU) wherever it fills the
        // device: 960 / 918 - 944 / 960 TFLOP/s on N x K = 4096x4096 / 11008x4096 / 4096x11008 at 2048 rows
        // (1050 - 1110 at 4096 rows), against 921 / 777 / 856 on the 128 x 128 tile (two workgroups a CU, bound by the
        // LDS port: 20 KB of operand reads and staging writes per 16 MFMAs and wave) and 750 - 760 on the 128 x 256
        // tile staged through registers (one wave per SIMD, nothing to run while it waits).
        // (512 rows x 22016 columns, the gate / up projection of a 512-token prompt: 117 us against 133)
        if (rows >= 512 && t_large >= cus) return launch_big<KIND, 2, 4, NEED_SUM>(p, stream);
        if (rows > 1024 && t_mid >= cus) return launch_big<KIND, 1, 4, NEED_SUM>(p, stream);
    } else {
        // 4-bit kinds: the same 128 x 256 tile (UINT4 850 / 922 / 916 TFLOP/s at 2048 rows on 4096^2, 11008 x 4096,
        // 4096 x 11008 against 785 / 743 / 861 staged through registers, one workgroup a CU; NF4 499 / 549 / 535
        // against 495 / 483 / 540).  The 128 x 128 tile (two workgroups a CU) measured no better than the staged
        // 128 x 256 one (UINT4 751 / 766 / 813, NF4 515 / 512 / 551).
        // (512 rows x 22016 columns: UINT4 119 us against 138, NF4 203 against 210)
        if (rows >= 512 && t_large >= cus) return launch_big<KIND, 2, 4, NEED_SUM>(p, stream);
    }
    if constexpr (KIND != XFTHIP_W_BF16) {
        // Few rows against a deep K (512 tokens x 4096 columns): 64-row tiles would leave one
        // workgroup per CU, whose k loop is then a chain of load latencies; 32-row tiles put two
        // on a CU.
        // (the K parts of a split GEMM count as workgroups of their own)
        if (t_small * (p.ksplit > 1 ? p.ksplit : 1) < 2 * cus) return launch_big<KIND, 1, 1, NEED_SUM>(p, stream);
        return launch_big<KIND, 1, 2, NEED_SUM>(p, stream);
    }
}

} // namespace
} // namespace xfthip
