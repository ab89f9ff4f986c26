// The lightning-indexer prolog's fixed-order sums over the hidden axis as wave jobs (decode forms): shared by the
// indexer prolog's first launch and by the fused prolog, whose matrix-core launch takes them along as riders.
#pragma once
#include "lip_kernels.h"
#include "prolog_common.h"

namespace pto {
namespace {

// Hidden-axis jobs: block c of 64 rows, tokens t0 .. t0+XTOK-1.  Even jobs take wk (lane l: columns 2l,
// 2l+1), odd jobs w_proj (lane l: column l).  The block of weights (contiguous in memory) travels to
// the wave's LDS region by LDS-DMA, the token slices are converted to fp32 on the way in; the
// product loop reads weights per lane and the hidden states as broadcasts.  XTOK = 2 gives a batch of up to
// eight tokens one job per wave of the launch; larger batches take 4 or 8 tokens per staged block, so that the
// launch stays one round of workgroups and a block is staged once per 4 or 8 tokens (the sums, one per token
// and column over ascending rows, do not depend on XTOK).
constexpr int XW_BYTES = LIP_XBLOCK * LIP_DIM * 2;     // 16 KiB: a block of wk
constexpr int XTOK_MAX = 8;                           // most tokens per hidden-axis job
constexpr int X_REGION_BYTES = XW_BYTES + XTOK_MAX * LIP_XBLOCK * 4;
constexpr int LIN_XWAVES = 4;

template <int XTOK>
__device__ __forceinline__ void x_linear_job(const LipParams &p, uint8_t *region, const int job)
{
    const int l = threadIdx.x & 63;
    const int nblk = p.h / LIP_XBLOCK;
    const int c = (job >> 1) % nblk;
    const int t0 = ((job >> 1) / nblk) * XTOK;
    const int k0 = c * LIP_XBLOCK;
    const bool proj = job & 1;
    const uint32_t wdst = (uint32_t)(uintptr_t)(lds_byte_t *)region;
    float *xs = reinterpret_cast<float *>(region + XW_BYTES);          // [XTOK][64]

    // the block: rows k0..k0+63 of wk (256 bytes each) or of w_proj (2*n_heads bytes each), contiguous
    const int bytes = proj ? LIP_XBLOCK * p.n_heads * 2 : XW_BYTES;
    const uint8_t *wsrc = proj ? reinterpret_cast<const uint8_t *>(p.w_proj) + (size_t)k0 * p.n_heads * 2
                               : reinterpret_cast<const uint8_t *>(p.wk) + (size_t)k0 * LIP_DIM * 2;
#pragma unroll 1
    for (int off = 0; off < bytes; off += 1024) {
        int o = off + 16 * l;
        o = o < bytes - 16 ? o : bytes - 16;            // lanes past the end re-read its last 16 bytes
        dma16(wsrc + o, wdst + off);
    }
#pragma unroll
    for (int tp = 0; tp < XTOK; tp += 2) {   // lane l: hidden states k0 + 2*(l%32), +1 of token t0 + tp + l/32
        const int t = t0 + tp + (l >> 5);
        const int tt = t < p.T ? t : p.T - 1;
        const uint32_t xv = reinterpret_cast<const uint32_t *>(p.x + (size_t)tt * p.h + k0)[l & 31];
        f32x2 v = {__uint_as_float(xv << 16), __uint_as_float(xv & 0xffff0000u)};
        *reinterpret_cast<f32x2 *>(xs + (tp + (l >> 5)) * LIP_XBLOCK + 2 * (l & 31)) = v;
    }
    VM_WAIT(0);
    // the wave reads back only what it wrote or requested itself: no barrier

    if (!proj) {
        const uint32_t *wl = reinterpret_cast<const uint32_t *>(region) + l;
        float a0[XTOK], a1[XTOK];
#pragma unroll
        for (int t = 0; t < XTOK; ++t) a0[t] = a1[t] = 0.f;
#pragma unroll 2
        for (int kk = 0; kk < LIP_XBLOCK; kk += 4) {
            f32x4 xv[XTOK];
#pragma unroll
            for (int t = 0; t < XTOK; ++t) xv[t] = *reinterpret_cast<const f32x4 *>(xs + t * LIP_XBLOCK + kk);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t wv = wl[(kk + j) * 64];
                const float w0 = __uint_as_float(wv << 16), w1 = __uint_as_float(wv & 0xffff0000u);
#pragma unroll
                for (int t = 0; t < XTOK; ++t) {
                    a0[t] = __builtin_fmaf(xv[t][j], w0, a0[t]);
                    a1[t] = __builtin_fmaf(xv[t][j], w1, a1[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < XTOK; ++t) {
            if (t0 + t < p.T) {
                f32x2 v = {a0[t], a1[t]};
                *reinterpret_cast<f32x2 *>(p.xpart + ((size_t)c * p.T + t0 + t) * LIP_XCOLS + 2 * l) = v;
            }
        }
    } else {
        const bool pl = l < p.n_heads;
        const uint16_t *wl = reinterpret_cast<const uint16_t *>(region) + (pl ? l : 0);
        float a2[XTOK];
#pragma unroll
        for (int t = 0; t < XTOK; ++t) a2[t] = 0.f;
#pragma unroll 2
        for (int kk = 0; kk < LIP_XBLOCK; kk += 4) {
            f32x4 xv[XTOK];
#pragma unroll
            for (int t = 0; t < XTOK; ++t) xv[t] = *reinterpret_cast<const f32x4 *>(xs + t * LIP_XBLOCK + kk);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float w2 = bf16_bits_to_f32(wl[(kk + j) * p.n_heads]);
#pragma unroll
                for (int t = 0; t < XTOK; ++t) a2[t] = __builtin_fmaf(xv[t][j], w2, a2[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < XTOK; ++t)
            if (t0 + t < p.T && pl) p.xpart[((size_t)c * p.T + t0 + t) * LIP_XCOLS + LIP_DIM + l] = a2[t];
    }
}

// tokens per hidden-axis job: 2 up to eight tokens, 4 up to sixteen, 8 beyond (a workgroup holds a compute unit, so
// more jobs than one round of workgroups has waves run as further rounds)
__host__ __device__ inline int lip_xtok(const int T) { return T <= 8 ? 2 : (T <= 16 ? 4 : 8); }
__host__ __device__ inline int lip_x_jobs(const LipParams &p, const int xtok) { return 2 * (p.h / LIP_XBLOCK) * ((p.T + xtok - 1) / xtok); }

// jobs first, first + stride, ... of a wave, xtok tokens per job (uniform)
__device__ __forceinline__ void x_linear_jobs(const LipParams &p, uint8_t *region, const int first, const int stride, const int x_jobs, const int xtok)
{
    if (xtok == 2) {
        for (int j = first; j < x_jobs; j += stride) x_linear_job<2>(p, region, j);
    } else if (xtok == 4) {
        for (int j = first; j < x_jobs; j += stride) x_linear_job<4>(p, region, j);
    } else {
        for (int j = first; j < x_jobs; j += stride) x_linear_job<8>(p, region, j);
    }
}

}  // namespace
}  // namespace pto
