// Prefill attention on 32 x 32 MFMA tiles: many (query token, query head) columns per (sequence, KV head).
//
// Replaces the reference's flash-style prefill (xft::selfScaledDpAttention, src/kernels/attention_kernels.h:1283-1408;
// DecoderUtil::incrementalTileAttention / softmaxTile / updateOutTile, src/utils/decoder_util.h:606-889) and its
// chunked prefill over a cache (xft::crossAttnByHead, attention_kernels.h:988-1123) when a launch has enough
// columns to fill the device.
//
// Why this shape.  A workgroup shares each 32-token block of keys and values through LDS, and every MFMA of a wave
// takes one operand from there.  The LDS port delivers 128 bytes a clock to the whole CU; a 16 x 16 x 32 MFMA
// (16 cycles) needs a 1 KiB operand, four SIMDs issuing them back to back would need 256 bytes a clock - the
// 16-column form is bound by the LDS port at half the MFMA rate before any softmax arithmetic.  A
// 32 x 32 x 16 MFMA (32 cycles) does twice the work on the same 1 KiB operand: the port and the MFMA pipes are
// in balance, and a wave owns 32 columns instead of 16, so a K / V byte is read from LDS half as often per flop.
//
//   S^T = K . Q^T   tile: 32 tokens (rows) x 32 columns; A = keys from LDS, B = the wave's queries, held in
//                   registers for the whole walk (8 k-steps of 16 dims)
//   O^T += V^T . P^T  4 tiles of 32 dims x 32 columns; A = values from LDS (token index innermost, as the cache
//                   stores them), B = probabilities straight from the score registers
// In the 32 x 32 accumulator a lane owns one column and 16 of the 32 rows (rows 8 q + 4 h + s; h = lane / 32,
// q = 0..3, s = 0..3), the other 16 sit in the lane 32 away.  The cache stores a value block with its tokens
// permuted (kvcache.h: 16-byte chunk c of a dim row = tokens 4 c .. 4 c + 3 and 16 + 4 c .. 16 + 4 c + 3); with the
// score rows in natural token order, chunk c = 2 t + h is exactly what lane half h holds in registers q = t and
// q = t + 2, so the probabilities of k-step t need no exchange between lanes.
//
// Online softmax per column in the log2 domain, fp32; the reference point moves only when a block's maximum
// exceeds it by more than 2^8 (probabilities up to 256 are exact enough in fp16 and in the fp32 sums), so the
// 64 accumulator registers of a lane are rescaled in few blocks only.  INT8 cache: codes are widened to fp16
// (exact) on their way into LDS, the key scale multiplies the score row, the value scale the probability; the
// value scales are taken relative to a running reference that is part of the same lazy rescaling (it moves when
// a block's largest scale leaves [ref / 1024, 4 ref]), so fp16 probabilities stay in range whatever the scales.
#pragma once
#include "attention_dev.h"

namespace xfthip {

constexpr int kP32ScaleBytes = 256; // 32 key scales + 32 value scales of a block (INT8 cache)
constexpr int kP32BufBytes = kPfBufBytes + kP32ScaleBytes;

union HFrag32 {
    f16x8 v;
    uint32_t u[4];
    u32x4 q;
};

// NW waves a workgroup, 32 columns a wave
// NW waves a workgroup, CT column tiles (32 CT columns) a wave; the library launches CT = 1, two workgroups a CU.
// Measured in that form (4 x 2048 tokens, 32 query / 8 KV heads, 213 us): the LDS pipe busy 90 % of the time (16
// operand reads and 4 staging writes a block and wave at about 22 cycles each), matrix pipes 29 %, vector ALUs 29 %;
// taking the MFMAs out of the kernel left 143 us, the softmax as well 119 us: the operand reads bound it.
// CT = 2 (every fragment read feeds two MFMAs; a wave then needs the registers of a whole SIMD, one workgroup a CU)
// halves the LDS bytes per flop but ran 353 us: a single wave a SIMD executes score MFMAs, softmax and value MFMAs
// strictly one after the other.  A three-stage software pipeline inside the wave (value MFMAs of block k - 1 and
// score MFMAs of block k + 1 issued between the softmax instructions of block k, the order fixed with scheduling
// fences) was built for both CT: correct, but 41 (CT = 1) and 182 (CT = 2) registers short, and the spill traffic
// shares the counter of the block prefetch, so every reload waited for it: 542 and 1560 us.  Requesting blocks two
// steps ahead, 8-wave workgroups and touching the pair's cache lines on arrival (L2 warm-up) each changed nothing:
// global latency and barriers are not what the waves wait for.  The LDS port itself, measured with a kernel of
// nothing but conflict-free 128-bit reads: 7.2 ns a wave-read a CU (about 140 bytes/ns; 64- and 32-bit reads move
// 75 - 80), so the 16 KB a wave reads per block put a floor of about 150 us under this shape.  Taking the value
// operands straight from the cache instead (they are laid out as the MFMA wants them; one block ahead, into the
// registers the products have just read: 209 registers) to share the bytes between the LDS port and the vector
// memory pipeline ran 262 us: a lane's 16 bytes lie 64 bytes from its neighbour's, and the memory pipeline serves
// such a load line by line.  What did pay for the FP16 cache: sending the blocks global -> LDS directly (below) instead
// of through registers and ds_write - 4 of a wave's 20 LDS instructions a block gone, 16 registers free: 213 -> 202 us.
// INT8 cache, measured and not kept: the block kept in LDS as codes (8 KB instead of 16), a lane's 128-bit read serving
// two k-steps (the queries' dims and, through a lane-half exchange, the probabilities' tokens permuted to match) -
// 8 operand reads a block and wave instead of 16, widened by every wave in registers: correct, and 354 us against
// 292: the 160 widening instructions a wave and block cost more than the LDS port had.
template <int NW, int CT, bool INT8>
__device__ inline void attn_prefill32_unit(const AttnParams &p, const int kvh, const int cgroup, const int b, unsigned char *lds) {
    constexpr int D = 128, NT = NW * 64, WC = 32 * CT;
    // FP16 cache, one tile a wave: reference point and row sums through the MFMAs (below); with two tiles a wave the
    // 64 registers this takes are not there, and the vector ALUs have the time
    constexpr bool VIA_MFMA = !INT8 && CT == 1;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, cl = lane & 31;
    int past = p.past;
    if (p.past_dev) {
        past = p.past_dev[b];
        past = past < 0 ? 0 : (past > p.kv.S - p.S ? p.kv.S - p.S : past);
    }
    past = __builtin_amdgcn_readfirstlane(past);
    const int ncols = p.S * p.G;
    const int c0 = (cgroup * NW + wave) * WC; // first column of this wave
    bool cvalid[CT];
    int cs[CT], cj[CT], limit[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int c = c0 + 32 * ct + cl;
        cvalid[ct] = c < ncols;
        cs[ct] = cvalid[ct] ? c / p.G : 0, cj[ct] = cvalid[ct] ? c % p.G : 0;
        limit[ct] = cvalid[ct] ? past + cs[ct] + 1 : 0; // tokens [0, limit) are visible to this column
    }
    const int lim_min = c0 + WC - 1 < ncols ? past + c0 / p.G + 1 : 0; // every column of the wave sees at least this many
    int wave_last = c0 + WC - 1;
    wave_last = wave_last < ncols ? wave_last : ncols - 1;
    const int wave_lim = c0 < ncols ? past + wave_last / p.G + 1 : 0; // no column of the wave sees a token from here on
    const int wave_nblk = (wave_lim + 31) >> 5;
    int wg_last = (cgroup + 1) * NW * WC - 1;
    wg_last = wg_last < ncols ? wg_last : ncols - 1;
    const int nblk = (past + wg_last / p.G + 1 + 31) >> 5;

    const size_t bh = (size_t)b * p.kv.H + kvh;
    constexpr int ESZ = INT8 ? 1 : 2;
    const ATTN_GLOBAL char *kbase = (const ATTN_GLOBAL char *)p.kv.k + bh * p.kv.S * D * ESZ;
    const ATTN_GLOBAL char *vbase = (const ATTN_GLOBAL char *)p.kv.v + bh * p.kv.S * D * ESZ;
    const ATTN_GLOBAL float *ksc = INT8 ? (const ATTN_GLOBAL float *)p.kv.kscale + bh * p.kv.S : nullptr;
    const ATTN_GLOBAL float *vsc = INT8 ? (const ATTN_GLOBAL float *)p.kv.vscale + bh * p.kv.S : nullptr;

    // ---- FP16 cache: the block copy global -> LDS without a stop in registers (global_load_lds_dwordx4: a wave
    // instruction fills 1 KiB of consecutive LDS, lane after lane, from 64 addresses of its choice).  Rows carry no
    // padding; the 16-byte chunk c of a key row (token r, 256 bytes) sits in slot c ^ (r & 15), of a value row (dim
    // r, 64 bytes) in slot c ^ ((r >> 2) & 3) - the lane fetches the global chunk that belongs in its slot - which
    // keeps the operand reads (32 rows, one chunk index) free of bank conflicts.  Three buffers of 16 KB: block
    // k + 2 is requested before block k is computed, and the barrier that ends a block first waits (vmcnt: the
    // requests retire in order) for the requests of the block before.  A wave sends requests 2 w, 2 w + 1 of the
    // keys' eight and of the values' eight.
    constexpr bool DIRECT = !INT8;
    constexpr int BUFB = DIRECT ? 16384 : kP32BufBytes, KPITCH = DIRECT ? 256 : kPfKPitch, VPITCH = DIRECT ? 64 : kPfVPitch;
    uint32_t rq_koff[2], rq_voff[2];
    const int wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = 2 * wave_u + i;
        const int kr = 4 * j + (lane >> 4), vr = 16 * j + (lane >> 2);
        rq_koff[i] = kr * 256 + (((lane & 15) ^ (kr & 15)) << 4);
        rq_voff[i] = vr * 64 + (((lane & 3) ^ ((vr >> 2) & 3)) << 4);
    }
    const uint32_t lds_rq = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds + 2048 * (uint32_t)wave_u;
    auto sgpr_ptr = [](const ATTN_GLOBAL char *ptr) { // the same in every lane; said so, for a scalar register pair
        const uint64_t bits = (uint64_t)(uintptr_t)ptr;
        return (const char *)(uintptr_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(bits >> 32)) << 32) |
                (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bits));
    };
    const char *k_uniform = sgpr_ptr(kbase), *v_uniform = sgpr_ptr(vbase);
    // (assembly, not the compiler's builtin for the instruction: after that one every later counted wait becomes a wait
    // for everything.  M0 carries the LDS address of the wave's first lane; one wait state between writing it and the
    // request.)
    auto request = [&](const int buf, const int blk_raw) {
        const int blk = __builtin_amdgcn_readfirstlane(blk_raw);
        const char *ks = k_uniform + (size_t)blk * (32 * D * 2), *vs = v_uniform + (size_t)blk * (32 * D * 2);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t kd = lds_rq + buf * BUFB + i * 1024, vd = kd + 8192;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(kd), "v"(rq_koff[i]), "s"(ks) : "memory");
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(vd), "v"(rq_voff[i]), "s"(vs) : "memory");
        }
    };

    // ---- INT8 cache: the block copy global -> registers -> LDS (widened on the way): 256 + 256 chunks of 16 bytes ----
    constexpr int CHUNKS = INT8 ? 256 : 512, PER = (CHUNKS + NT - 1) / NT;
    u32x4 kstage[PER], vstage[PER];
    f32x4 sstage; // INT8: threads 0..7 carry 4 key scales each, threads 8..15 4 value scales
    auto fetch = [&](const int blk) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int ch = threadIdx.x + NT * i;
            if (CHUNKS % NT == 0 || ch < CHUNKS) {
                kstage[i] = *(const ATTN_GLOBAL u32x4 *)(kbase + (size_t)blk * (32 * D * ESZ) + (size_t)ch * 16);
                vstage[i] = *(const ATTN_GLOBAL u32x4 *)(vbase + (size_t)blk * (32 * D * ESZ) + (size_t)ch * 16);
            }
        }
        if constexpr (INT8) {
            if (threadIdx.x < 16) sstage = *(const ATTN_GLOBAL f32x4 *)((threadIdx.x < 8 ? ksc : vsc) + (blk << 5) + 4 * (threadIdx.x & 7));
        }
    };
    auto widen16 = [&](const u32x4 raw, u32x4 &lo, u32x4 &hi) {
        HFrag x, y;
        widen_i8x4(raw[0], x.h[0], x.h[1]);
        widen_i8x4(raw[1], x.h[2], x.h[3]);
        widen_i8x4(raw[2], y.h[0], y.h[1]);
        widen_i8x4(raw[3], y.h[2], y.h[3]);
        lo = x.q, hi = y.q;
    };
    auto stash = [&](const int buf) {
        unsigned char *kb = lds + buf * kP32BufBytes, *vb = kb + 32 * kPfKPitch;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int ch = threadIdx.x + NT * i;
            if (CHUNKS % NT == 0 || ch < CHUNKS) {
                if constexpr (INT8) {
                    u32x4 lo, hi;
                    widen16(kstage[i], lo, hi); // token ch / 8, dims 16 (ch % 8) ..
                    *(u32x4 *)(kb + (ch >> 3) * kPfKPitch + (ch & 7) * 32) = lo;
                    *(u32x4 *)(kb + (ch >> 3) * kPfKPitch + (ch & 7) * 32 + 16) = hi;
                    widen16(vstage[i], lo, hi); // dim ch / 2, token slots 16 (ch % 2) ..
                    *(u32x4 *)(vb + (ch >> 1) * kPfVPitch + (ch & 1) * 32) = lo;
                    *(u32x4 *)(vb + (ch >> 1) * kPfVPitch + (ch & 1) * 32 + 16) = hi;
                } else {
                    *(u32x4 *)(kb + (ch >> 4) * kPfKPitch + (ch & 15) * 16) = kstage[i]; // token ch / 16, dims 8 (ch % 16) ..
                    *(u32x4 *)(vb + (ch >> 2) * kPfVPitch + (ch & 3) * 16) = vstage[i]; // dim ch / 4, tokens 8 (ch % 4) ..
                }
            }
        }
        if constexpr (INT8) {
            if (threadIdx.x < 16) *(f32x4 *)(kb + kPfBufBytes + 16 * threadIdx.x) = sstage;
        }
    };

    // ---- this wave's queries: B operand of the score MFMA, k-step s covers dims 16 s + 8 h .. + 8 ----
    // FP16 cache: the queries carry the softmax scale and log2 e (rounded to fp16 once: 2^-12 relative, the size of
    // the rounding of the fp16 probabilities), so that a score leaves the MFMA in the log2 domain.
    const float c1 = p.scale * 1.4426950408889634f;
    const float qmul = INT8 ? 1.0f : c1;
    HFrag32 qf[CT][8];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const uint16_t *qrow = p.q + ((size_t)b * p.S + cs[ct]) * p.qStride + (size_t)(kvh * p.G + cj[ct]) * D;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint32_t raw[4] = {0u, 0u, 0u, 0u};
            if (cvalid[ct]) ld_dev16(qrow + 16 * s + 8 * h, raw);
#pragma unroll
            for (int i = 0; i < 4; ++i) qf[ct][s].u[i] = pack_f16(u2f(raw[i] << 16) * qmul, u2f(raw[i] & 0xFFFF0000u) * qmul);
        }
    }
    float m_run[CT], l_run[CT]; // m_run == kNegBig: the column has seen no token yet
    float vref = 0.0f; // INT8: the value scales are taken relative to this (0 = not set yet)
    f32x16 o[CT][4];
    // FP16 cache: the score MFMAs start from -m_run instead of 0, so a score arrives relative to the column's
    // reference point with no vector instruction spent on it, and the row sums of the probabilities come out of
    // two more MFMAs against a tile of ones (the matrix pipes have the slack, the vector ALUs do not).
    f32x16 negm[VIA_MFMA ? CT : 1], lacc[VIA_MFMA ? CT : 1];
    HFrag32 ones;
#pragma unroll
    for (int r = 0; r < 16; ++r) negm[0][r] = 0.0f, lacc[0][r] = 0.0f;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        m_run[ct] = kNegBig, l_run[ct] = 0.0f;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) o[ct][dt] = negm[0];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) ones.u[i] = 0x3C003C00u;

    auto compute = [&](const int buf, const int blk) {
        const int t0 = blk << 5;
        const unsigned char *kb = lds + buf * BUFB, *vb = kb + 32 * KPITCH;
        const unsigned char *krow = kb + cl * KPITCH + (DIRECT ? 0 : 16 * h);
        HFrag32 kf[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) kf[s].q = *(const u32x4 *)(krow + (DIRECT ? (((2 * s + h) ^ (cl & 15)) << 4) : 32 * s));
        f32x16 sc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if constexpr (!VIA_MFMA) {
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[ct][r] = 0.0f;
            } else {
                sc[ct] = negm[ct];
            }
        }
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) sc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s].v, qf[ct][s].v, sc[ct], 0, 0, 0);
        // the value operands are read only now: they reuse the key operands' registers and their LDS latency
        // passes behind the softmax arithmetic
        __builtin_amdgcn_sched_barrier(0);
        HFrag32 vf[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
                vf[t][dt].q = *(const u32x4 *)(vb + (32 * dt + cl) * VPITCH + (DIRECT ? (((2 * t + h) ^ ((cl >> 2) & 3)) << 4) : 16 * (2 * t + h)));
        const bool masked = t0 + 32 > lim_min; // wave-uniform
        // INT8: scales of this lane's 16 tokens (8 q + 4 h ..)
        f32x4 ks[4], vs[4];
        float vmax = 0.0f, vinv = 1.0f, vmove = 1.0f;
        if constexpr (INT8) {
            const float *sl = (const float *)(kb + kPfBufBytes);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                ks[q] = *(const f32x4 *)(sl + 8 * q + 4 * h) * c1; // key scale and softmax scale in one factor
                vs[q] = *(const f32x4 *)(sl + 32 + 8 * q + 4 * h);
                // (tokens no column of the wave sees stay out: behind the sequence's end the cache may hold anything)
#pragma unroll
                for (int r = 0; r < 4; ++r) vmax = fmaxf(vmax, t0 + 8 * q + 4 * h + r < wave_lim ? vs[q][r] : 0.0f);
            }
            vmax = fmaxf(vmax, swap32(vmax)); // the block's largest value scale, the same in every lane
            // value scales relative to vref; vref follows the blocks' largest scale lazily, like the maximum
            if (vmax > 4.0f * vref || (vmax > 0.0f && vmax * 1024.0f < vref)) { // wave-uniform
                vmove = vref > 0.0f ? vref / vmax : 1.0f;
                vref = vmax;
            }
            vinv = vref > 0.0f ? 1.0f / vref : 0.0f;
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x16 &x = sc[ct];
            float pr[16];
            if constexpr (!VIA_MFMA) {
                if constexpr (INT8) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] *= ks[r >> 2][r & 3];
                }
                if (masked) {
                    // only the blocks on the causal diagonal pay for the mask (a real branch)
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = (t0 + 8 * (r >> 2) + 4 * h + (r & 3)) < limit[ct] ? x[r] : kNegBig;
                }
                float bmax = fmaxf(fmaxf(x[0], x[1]), x[2]);
#pragma unroll
                for (int r = 3; r < 15; r += 2) bmax = fmaxf(fmaxf(bmax, x[r]), x[r + 1]);
                bmax = fmaxf(bmax, x[15]);
                bmax = fmaxf(bmax, swap32(bmax));
                const float m_new = bmax > m_run[ct] + 8.0f ? bmax : m_run[ct];
                const float alpha = __builtin_amdgcn_exp2f(m_run[ct] - m_new);
                m_run[ct] = m_new;
#pragma unroll
                for (int r = 0; r < 16; ++r) pr[r] = __builtin_amdgcn_exp2f(x[r] - m_new);
                if (masked) {
                    // a masked score is kNegBig: 2^(kNegBig - m) is already 0 unless the column has seen nothing yet
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int r = 0; r < 16; ++r) pr[r] = x[r] > 0.5f * kNegBig ? pr[r] : 0.0f;
                }
                float psum = (pr[0] + pr[1]) + (pr[2] + pr[3]);
#pragma unroll
                for (int r = 4; r < 16; r += 4) psum += (pr[r] + pr[r + 1]) + (pr[r + 2] + pr[r + 3]);
                l_run[ct] = l_run[ct] * alpha + psum; // (this lane's 16 rows; the two halves are added at the end)
                const float oscale = alpha * vmove; // what the running output is multiplied by before this block is added
                if constexpr (INT8) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) pr[r] *= vs[r >> 2][r & 3] * vinv;
                }
                if (__builtin_amdgcn_ballot_w64(oscale != 1.0f) != 0) {
                    // the running output is rescaled only when some column's reference point moved (a real branch)
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o[ct][dt][r] *= oscale;
                }
            } else {
                if (masked) {
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = (t0 + 8 * (r >> 2) + 4 * h + (r & 3)) < limit[ct] ? x[r] : kNegBig;
                }
                // x = log2-domain score minus the column's reference point (0 while the column has seen nothing)
                float bmax = fmaxf(fmaxf(x[0], x[1]), x[2]);
#pragma unroll
                for (int r = 3; r < 15; r += 2) bmax = fmaxf(fmaxf(bmax, x[r]), x[r + 1]);
                bmax = fmaxf(bmax, x[15]);
                bmax = fmaxf(bmax, swap32(bmax));
                // the reference point moves when the block's maximum exceeds it by more than 2^8, and is set by the
                // first block a column sees anything of
                const bool first = m_run[ct] == kNegBig;
                const bool move = bmax > 8.0f || (first && bmax > 0.5f * kNegBig);
                if (__builtin_amdgcn_ballot_w64(move) != 0) {
                    // a real branch: in most blocks no column of the wave moves
                    asm volatile("" ::: "memory");
                    const float delta = move ? bmax : 0.0f;
                    const float alpha = __builtin_amdgcn_exp2f(-delta); // (columns that see their first tokens hold zeros)
                    if (move) m_run[ct] = (first ? 0.0f : m_run[ct]) + delta;
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] -= delta, negm[ct][r] = move ? -m_run[ct] : negm[ct][r], lacc[ct][r] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o[ct][dt][r] *= alpha;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) pr[r] = __builtin_amdgcn_exp2f(x[r]); // (a masked score is kNegBig: 0)
            }
            HFrag32 pf[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                pf[t].u[0] = pack_f16(pr[4 * t], pr[4 * t + 1]);
                pf[t].u[1] = pack_f16(pr[4 * t + 2], pr[4 * t + 3]);
                pf[t].u[2] = pack_f16(pr[4 * t + 8], pr[4 * t + 9]);
                pf[t].u[3] = pack_f16(pr[4 * t + 10], pr[4 * t + 11]);
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int dt = 0; dt < 4; ++dt) o[ct][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[t][dt].v, pf[t].v, o[ct][dt], 0, 0, 0);
                if constexpr (VIA_MFMA) lacc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones.v, pf[t].v, lacc[ct], 0, 0, 0);
            }
        }
    };

    if constexpr (DIRECT) {
        if (nblk > 0) request(0, 0);
        if (nblk > 1) request(1, 1);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        int cur = 0;
        for (int blk = 0; blk < nblk; ++blk) {
            const bool more = blk + 2 < nblk; // uniform over the workgroup
            // (the buffer it goes to held block blk - 1, which every wave has left behind at the last barrier)
            if (more) request(cur == 0 ? 2 : cur - 1, blk + 2);
            if (blk < wave_nblk) compute(cur, blk);
            __builtin_amdgcn_sched_barrier(0);
            // block blk + 1 (requested an iteration ago: everything but this iteration's four requests) is in, and
            // this wave's reads of block blk are done
            if (more) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            cur = cur == 2 ? 0 : cur + 1;
        }
    } else {
    if (nblk > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();
    for (int blk = 0; blk < nblk; ++blk) {
        const bool more = blk + 1 < nblk; // uniform over the workgroup
        if (more) fetch(blk + 1);
        if (blk < wave_nblk) compute(blk & 1, blk);
        if (more) stash((blk + 1) & 1);
        __syncthreads();
    }
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        float l = l_run[ct];
        l += swap32(l);
        if constexpr (VIA_MFMA) l = lacc[ct][0]; // every row of the ones tile holds the column's sum over all tokens
        if (!cvalid[ct]) continue;
        const float inv = (INT8 ? vref : 1.0f) / l;
        const size_t base = ((size_t)b * p.S + cs[ct]) * p.oStride + (size_t)(kvh * p.G + cj[ct]) * D;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const size_t idx = base + 32 * dt + 8 * q + 4 * h;
                const float v0 = o[ct][dt][4 * q] * inv, v1 = o[ct][dt][4 * q + 1] * inv, v2 = o[ct][dt][4 * q + 2] * inv,
                            v3 = o[ct][dt][4 * q + 3] * inv;
                if (p.out_dtype == XFTHIP_BF16) {
                    const uint32_t lo = f32_to_bf16_ref(v0) | ((uint32_t)f32_to_bf16_ref(v1) << 16);
                    const uint32_t hi = f32_to_bf16_ref(v2) | ((uint32_t)f32_to_bf16_ref(v3) << 16);
                    uint16_t *dst = (uint16_t *)p.out + idx;
                    if ((((uintptr_t)dst) & 7) == 0) {
                        *(uint2 *)dst = make_uint2(lo, hi);
                    } else {
                        dst[0] = (uint16_t)lo, dst[1] = (uint16_t)(lo >> 16), dst[2] = (uint16_t)hi, dst[3] = (uint16_t)(hi >> 16);
                    }
                } else {
                    float *dst = (float *)p.out + idx;
                    dst[0] = v0, dst[1] = v1, dst[2] = v2, dst[3] = v3;
                }
            }
    }
}

} // namespace xfthip
