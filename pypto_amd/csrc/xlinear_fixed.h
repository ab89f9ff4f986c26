// Fixed-order sums over the hidden axis, one group of eight blocks of 64 rows per workgroup: x [T, h] bf16 times a
// slab of up to 128 columns of a row-major bf16 weight matrix.  Shared by the MLA prolog (w_dq, w_dkv_kr; every
// size) and the lightning-indexer prolog (wk, w_proj; prefill sizes); included after prolog_common.h.
//
// Every product of two bf16 values is exact in fp32; a block is summed ascending from 0.0 by fp32 FMAs, the
// workgroup's eight block sums (one per wave) meet in LDS and are added ascending into the group sum, which is all
// that reaches memory: out[t * out_pitch + column].  The caller adds the group sums ascending.
//   workgroup = (slab, group of 512 hidden rows, 8 tokens), eight waves; wave w takes block 8*group + w: the block
//   of the slab travels to the wave's LDS region by LDS-DMA, the hidden states are widened to fp32 on the way in,
//   the product loop reads weights per lane (columns 2l, 2l+1) and the hidden states as broadcasts.
#pragma once
#include "prolog_common.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

constexpr int XL_BLOCK = 64;                                           // rows per block
constexpr int XL_GROUP = 8;                                            // blocks per group
constexpr int XL_TOK = 8;                                              // tokens per workgroup
constexpr int XL_WAVES = XL_GROUP;                                     // one block per wave
constexpr int XL_W_BYTES = XL_BLOCK * 256;                             // a block of one slab: 64 rows x 256 bytes
constexpr int XL_REGION = XL_W_BYTES + XL_TOK * XL_BLOCK * 4;          // + the hidden states as fp32
constexpr int XL_LDS = XL_WAVES * XL_REGION;

struct XlSlab {
    const uint8_t *w;     // column 0 of the slab in row 0 of the weight matrix
    int pitch;            // bytes between rows of the weight matrix
    int wbytes;           // bytes of a row that belong to the slab: 16, 32, 64, 128 or 256
    float *out;           // group sums of this group: out[t * out_pitch + column of the slab]
    int out_pitch;
};

// row widths the staging handles (whole 16-byte pieces, a power of two of them per row)
__host__ __device__ inline bool xl_width_ok(const int wbytes) { return wbytes >= 16 && wbytes <= 256 && (wbytes & (wbytes - 1)) == 0; }

// group g of the hidden axis, tokens t0 .. t0 + 7 (rows past T - 1 repeat it and are not stored)
__device__ __forceinline__ void xl_body(const XlSlab &sl, const uint16_t *x, const int T, const int h, const int g, const int t0, uint8_t *smem)
{
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = h / XL_BLOCK;
    const int wbytes = sl.wbytes;

    uint8_t *region = smem + w * XL_REGION;
    float *xs = reinterpret_cast<float *>(region + XL_W_BYTES);         // [8][64]
    const int c = g * XL_GROUP + w;                                       // this wave's block
    const int nb = nblk - g * XL_GROUP < XL_GROUP ? nblk - g * XL_GROUP : XL_GROUP;
    float a0[XL_TOK], a1[XL_TOK];
#pragma unroll
    for (int t = 0; t < XL_TOK; ++t) a0[t] = a1[t] = 0.f;

    if (w < nb) {
        const int k0 = c * XL_BLOCK;
        const uint32_t wdst = (uint32_t)(uintptr_t)(lds_byte_t *)region;
        {   // rows of wbytes bytes: wbytes/16 lanes per row
            const int lpr = wbytes >> 4;
            const int rpi = 64 / lpr;                                     // rows per request
            const uint8_t *src = sl.w + (size_t)(k0 + l / lpr) * sl.pitch + 16 * (l % lpr);
#pragma unroll 1
            for (int i = 0; i < XL_BLOCK / rpi; ++i) dma16(src + (size_t)i * rpi * sl.pitch, wdst + 1024 * i);
        }
#pragma unroll
        for (int u = 0; u < XL_TOK / 2; ++u) {   // lane l: hidden states k0 + 2*(l%32), +1 of token t0 + 2u + l/32
            const int t = t0 + 2 * u + (l >> 5);
            const int tt = t < T ? t : T - 1;
            const uint32_t xv = reinterpret_cast<const uint32_t *>(x + (size_t)tt * h + k0)[l & 31];
            f32x2 v = {__uint_as_float(xv << 16), __uint_as_float(xv & 0xffff0000u)};
            *reinterpret_cast<f32x2 *>(xs + (2 * u + (l >> 5)) * XL_BLOCK + 2 * (l & 31)) = v;
        }
        VM_WAIT(0);
        const int rowdw = wbytes >> 2;
        const uint32_t *wl = reinterpret_cast<const uint32_t *>(region) + (l & (rowdw - 1));   // lanes past the slab's width repeat earlier ones
#pragma unroll 2
        for (int kk = 0; kk < XL_BLOCK; kk += 4) {
            f32x4 xv[XL_TOK];
#pragma unroll
            for (int t = 0; t < XL_TOK; ++t) xv[t] = *reinterpret_cast<const f32x4 *>(xs + t * XL_BLOCK + kk);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t wv = wl[(kk + j) * rowdw];
                const float w0 = __uint_as_float(wv << 16), w1 = __uint_as_float(wv & 0xffff0000u);
#pragma unroll
                for (int t = 0; t < XL_TOK; ++t) {
                    a0[t] = __builtin_fmaf(xv[t][j], w0, a0[t]);
                    a1[t] = __builtin_fmaf(xv[t][j], w1, a1[t]);
                }
            }
        }
        // block sums into this wave's own (consumed) region: [8 tokens][128 columns]
        float *bs = reinterpret_cast<float *>(region);
#pragma unroll
        for (int t = 0; t < XL_TOK; ++t) {
            f32x2 v = {a0[t], a1[t]};
            *reinterpret_cast<f32x2 *>(bs + t * 128 + 2 * l) = v;
        }
    }
    __syncthreads();
    // group sum: thread (token = w, columns 2l, 2l+1) chains the block sums in ascending order
    {
        const int t = t0 + w;
        const int width = wbytes >> 1;                                    // columns of the slab
        if (t < T && 2 * l < width) {
            float s0 = 0.f, s1 = 0.f;
            for (int i = 0; i < nb; ++i) {
                const f32x2 v = *reinterpret_cast<const f32x2 *>(reinterpret_cast<const float *>(smem + i * XL_REGION) + w * 128 + 2 * l);
                s0 = __fadd_rn(s0, v[0]);
                s1 = __fadd_rn(s1, v[1]);
            }
            f32x2 v = {s0, s1};
            *reinterpret_cast<f32x2 *>(sl.out + (size_t)t * sl.out_pitch + 2 * l) = v;
        }
    }
}

}  // namespace
}  // namespace pto
