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
    // xl_body only: a 256-byte slab may be two 128-byte halves of different matrices.  With w_hi set (wbytes = 256),
    // bytes 128..255 of a staged row are bytes 0..127 of w_hi's row, and columns 64..127 go to out_hi[t * out_pitch_hi + column - 64].
    const uint8_t *w_hi = nullptr;
    int pitch_hi = 0;
    float *out_hi = nullptr;
    int out_pitch_hi = 0;
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
            const bool hi = sl.w_hi != nullptr && (l & 15) >= 8;          // this lane's piece belongs to the second matrix
            const size_t pitch = hi ? sl.pitch_hi : sl.pitch;
            const uint8_t *src = (hi ? sl.w_hi - 128 : sl.w) + (size_t)(k0 + l / lpr) * pitch + 16 * (l % lpr);
#pragma unroll 1
            for (int i = 0; i < XL_BLOCK / rpi; ++i) dma16(src + (size_t)i * rpi * pitch, wdst + 1024 * i);
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
            float *dst = sl.out + (size_t)t * sl.out_pitch + 2 * l;
            if (sl.w_hi != nullptr && l >= 32) dst = sl.out_hi + (size_t)t * sl.out_pitch_hi + 2 * l - 64;
            *reinterpret_cast<f32x2 *>(dst) = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The same sums for prefill-sized token counts with the hidden states broadcast by the multiply-add itself: a lane
// keeps x[t][k0 + 2*(l % 16)] and x[t][k0 + 2*(l % 16) + 1] of a 32-row half block in two registers per token (every
// row of 16 lanes holds the same 32 values), and v_fmac_f32 with the DPP control row_newbcast:n reads lane n of the
// row, i.e. hidden row k0 + 2n (or + 1), in all lanes -- no LDS read and no extra instruction per hidden state, where
// the form above spends an LDS broadcast of 16 bytes per four multiply-adds.  Same products, same order (a block
// ascending from 0.0, the eight block sums ascending), so the same bits.
//   workgroup = (slab, group of 512 hidden rows, XD_TOK tokens), eight waves, wave w takes block 8*group + w.
//   PAIR: lane l holds columns 2l, 2l+1 (a slab of 128 columns); otherwise column l (a slab of up to 64).
constexpr int XD_TOK = 16;
constexpr int XD_LDS = XL_WAVES * XL_W_BYTES;

// acc[t] += bcast_N(x[t]) * w for eight tokens (and a second column with w1), as one statement: nothing the compiler
// emits can sit between the multiply-adds, and the statement opens with the two wait states a DPP read wants after a
// write of its operand, whatever the compiler did to these registers just before.
#define XD_F "v_fmac_f32_dpp %"
#define XD_B " row_newbcast:%[n] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
template <int N>
__device__ __forceinline__ void fmac8_pair(float *a0, float *a1, const float *x, const float w0, const float w1)
{
    asm("s_nop 1\n\t"
        XD_F "0, %16, %[w0]" XD_B XD_F "8, %16, %[w1]" XD_B XD_F "1, %17, %[w0]" XD_B XD_F "9, %17, %[w1]" XD_B
        XD_F "2, %18, %[w0]" XD_B XD_F "10, %18, %[w1]" XD_B XD_F "3, %19, %[w0]" XD_B XD_F "11, %19, %[w1]" XD_B
        XD_F "4, %20, %[w0]" XD_B XD_F "12, %20, %[w1]" XD_B XD_F "5, %21, %[w0]" XD_B XD_F "13, %21, %[w1]" XD_B
        XD_F "6, %22, %[w0]" XD_B XD_F "14, %22, %[w1]" XD_B XD_F "7, %23, %[w0]" XD_B XD_F "15, %23, %[w1]" XD_B
        : "+v"(a0[0]), "+v"(a0[1]), "+v"(a0[2]), "+v"(a0[3]), "+v"(a0[4]), "+v"(a0[5]), "+v"(a0[6]), "+v"(a0[7]),
          "+v"(a1[0]), "+v"(a1[1]), "+v"(a1[2]), "+v"(a1[3]), "+v"(a1[4]), "+v"(a1[5]), "+v"(a1[6]), "+v"(a1[7])
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]), [w0] "v"(w0), [w1] "v"(w1), [n] "n"(N));
}
template <int N>
__device__ __forceinline__ void fmac8_single(float *a0, const float *x, const float w0)
{
    asm("s_nop 1\n\t"
        XD_F "0, %8, %[w0]" XD_B XD_F "1, %9, %[w0]" XD_B XD_F "2, %10, %[w0]" XD_B XD_F "3, %11, %[w0]" XD_B
        XD_F "4, %12, %[w0]" XD_B XD_F "5, %13, %[w0]" XD_B XD_F "6, %14, %[w0]" XD_B XD_F "7, %15, %[w0]" XD_B
        : "+v"(a0[0]), "+v"(a0[1]), "+v"(a0[2]), "+v"(a0[3]), "+v"(a0[4]), "+v"(a0[5]), "+v"(a0[6]), "+v"(a0[7])
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]), [w0] "v"(w0), [n] "n"(N));
}
#undef XD_F
#undef XD_B

template <bool PAIR, int N>
__device__ __forceinline__ void xd_pair_of_rows(const uint8_t *wrow, const int rowbytes, const int lane_off, float (&xe)[XD_TOK],
                                                float (&xo)[XD_TOK], float (&a0)[XD_TOK], float (&a1)[XD_TOK])
{
#pragma unroll
    for (int odd = 0; odd < 2; ++odd) {
        float *xs = odd ? xo : xe;
        if (PAIR) {
            const uint32_t wv = *reinterpret_cast<const uint32_t *>(wrow + (2 * N + odd) * rowbytes + lane_off);
            const float w0 = __uint_as_float(wv << 16), w1 = __uint_as_float(wv & 0xffff0000u);
#pragma unroll
            for (int t = 0; t < XD_TOK; t += 8) fmac8_pair<N>(a0 + t, a1 + t, xs + t, w0, w1);
        } else {
            const float w0 = __uint_as_float((uint32_t) * reinterpret_cast<const uint16_t *>(wrow + (2 * N + odd) * rowbytes + lane_off) << 16);
#pragma unroll
            for (int t = 0; t < XD_TOK; t += 8) fmac8_single<N>(a0 + t, xs + t, w0);
        }
    }
}

template <bool PAIR>
__device__ __forceinline__ void xd_body(const XlSlab &sl, const uint16_t *x, const int T, const int h, const int g, const int t0, uint8_t *smem)
{
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = h / XL_BLOCK;
    const int wbytes = sl.wbytes;
    const int ncols = wbytes >> 1;
    uint8_t *region = smem + w * XL_W_BYTES;
    const int c = g * XL_GROUP + w;                                       // this wave's block
    const int nb = nblk - g * XL_GROUP < XL_GROUP ? nblk - g * XL_GROUP : XL_GROUP;
    float a0[XD_TOK], a1[XD_TOK];
#pragma unroll
    for (int t = 0; t < XD_TOK; ++t) a0[t] = a1[t] = 0.f;

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
        // hidden states of both half blocks: lane l holds rows k0 + 32*hb + 2*(l%16), +1 of every token
        uint32_t xr[2][XD_TOK];
#pragma unroll
        for (int hb = 0; hb < 2; ++hb)
#pragma unroll
            for (int t = 0; t < XD_TOK; ++t) {
                const int tt = t0 + t < T ? t0 + t : T - 1;
                xr[hb][t] = reinterpret_cast<const uint32_t *>(x + (size_t)tt * h + k0 + 32 * hb)[l & 15];
            }
        VM_WAIT(0);
        const int lane_off = PAIR ? 4 * (2 * l < ncols ? l : 0) : 2 * (l < ncols ? l : 0);
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            float xe[XD_TOK], xo[XD_TOK];
#pragma unroll
            for (int t = 0; t < XD_TOK; ++t) {
                xe[t] = __uint_as_float(xr[hb][t] << 16);
                xo[t] = __uint_as_float(xr[hb][t] & 0xffff0000u);
            }
            const uint8_t *wrow = region + 32 * hb * wbytes;
            xd_pair_of_rows<PAIR, 0>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 1>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 2>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 3>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 4>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 5>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 6>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 7>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 8>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 9>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 10>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 11>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 12>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 13>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 14>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            xd_pair_of_rows<PAIR, 15>(wrow, wbytes, lane_off, xe, xo, a0, a1);
        }
    }
    __syncthreads();                                   // every wave is done with its block of weights
    // block sums into this wave's own (consumed) region: [XD_TOK tokens][128 columns]
    if (w < nb) {
        float *bs = reinterpret_cast<float *>(region);
#pragma unroll
        for (int t = 0; t < XD_TOK; ++t) {
            if (PAIR) {
                f32x2 v = {a0[t], a1[t]};
                *reinterpret_cast<f32x2 *>(bs + t * 128 + 2 * l) = v;
            } else {
                bs[t * 128 + l] = a0[t];
            }
        }
    }
    __syncthreads();
    // group sums: wave w chains the block sums of tokens w and w + 8 in ascending order
#pragma unroll
    for (int u = 0; u < XD_TOK / XL_WAVES; ++u) {
        const int tl = w + XL_WAVES * u;
        const int t = t0 + tl;
        if (t < T) {
            if (PAIR) {
                if (2 * l < ncols) {
                    float s0 = 0.f, s1 = 0.f;
                    for (int i = 0; i < nb; ++i) {
                        const f32x2 v = *reinterpret_cast<const f32x2 *>(reinterpret_cast<const float *>(smem + i * XL_W_BYTES) + tl * 128 + 2 * l);
                        s0 = __fadd_rn(s0, v[0]);
                        s1 = __fadd_rn(s1, v[1]);
                    }
                    f32x2 v = {s0, s1};
                    *reinterpret_cast<f32x2 *>(sl.out + (size_t)t * sl.out_pitch + 2 * l) = v;
                }
            } else if (l < ncols) {
                float s0 = 0.f;
                for (int i = 0; i < nb; ++i) s0 = __fadd_rn(s0, reinterpret_cast<const float *>(smem + i * XL_W_BYTES)[tl * 128 + l]);
                sl.out[(size_t)t * sl.out_pitch + l] = s0;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The DPP form for a slab of 64 columns in a workgroup of FOUR waves, so that its jobs can ride in a launch whose
// workgroups have 256 threads: wave w takes blocks w and w + 4 of the group one after the other (the same 64
// sequential multiply-adds per block from 0.0), the eight block sums are parked in LDS beside the staging areas and
// chained ascending into the group sum -- product by product and sum by sum what xd_body<false> computes, so the
// same bits.  LDS: four staging areas of 64 rows x 128 bytes, then eight block-sum areas of [XD_TOK][64] floats.
constexpr int XR_WAVES = 4;
constexpr int XR_STAGE = XL_BLOCK * 128;                                 // a block of the slab: 64 rows x 128 bytes
constexpr int XR_SUMS = XD_TOK * 64 * 4;
constexpr int XR_LDS = XR_WAVES * XR_STAGE + XL_GROUP * XR_SUMS;

__device__ __forceinline__ void xr_body(const XlSlab &sl, const uint16_t *x, const int T, const int h, const int g, const int t0, uint8_t *smem)
{
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nblk = h / XL_BLOCK;
    constexpr int wbytes = 128;
    uint8_t *region = smem + w * XR_STAGE;
    const int nb = nblk - g * XL_GROUP < XL_GROUP ? nblk - g * XL_GROUP : XL_GROUP;
#pragma unroll 1
    for (int pass = 0; pass < XL_GROUP / XR_WAVES; ++pass) {
        const int bi = w + XR_WAVES * pass;                               // this wave's block of the group
        if (bi < nb) {
            float a0[XD_TOK], a1[XD_TOK];
#pragma unroll
            for (int t = 0; t < XD_TOK; ++t) a0[t] = a1[t] = 0.f;
            const int k0 = (g * XL_GROUP + bi) * XL_BLOCK;
            const uint32_t wdst = (uint32_t)(uintptr_t)(lds_byte_t *)region;
            {   // rows of 128 bytes: eight lanes per row, eight rows per request
                const uint8_t *src = sl.w + (size_t)(k0 + (l >> 3)) * sl.pitch + 16 * (l & 7);
#pragma unroll 1
                for (int i = 0; i < XL_BLOCK / 8; ++i) dma16(src + (size_t)i * 8 * sl.pitch, wdst + 1024 * i);
            }
            uint32_t xr[2][XD_TOK];
#pragma unroll
            for (int hb = 0; hb < 2; ++hb)
#pragma unroll
                for (int t = 0; t < XD_TOK; ++t) {
                    const int tt = t0 + t < T ? t0 + t : T - 1;
                    xr[hb][t] = reinterpret_cast<const uint32_t *>(x + (size_t)tt * h + k0 + 32 * hb)[l & 15];
                }
            VM_WAIT(0);
            const int lane_off = 2 * l;
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) {
                float xe[XD_TOK], xo[XD_TOK];
#pragma unroll
                for (int t = 0; t < XD_TOK; ++t) {
                    xe[t] = __uint_as_float(xr[hb][t] << 16);
                    xo[t] = __uint_as_float(xr[hb][t] & 0xffff0000u);
                }
                const uint8_t *wrow = region + 32 * hb * wbytes;
                xd_pair_of_rows<false, 0>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 1>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 2>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 3>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 4>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 5>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 6>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 7>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 8>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 9>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 10>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 11>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 12>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 13>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 14>(wrow, wbytes, lane_off, xe, xo, a0, a1);
                xd_pair_of_rows<false, 15>(wrow, wbytes, lane_off, xe, xo, a0, a1);
            }
            // (the LDS reads of the weights above are complete: their results were consumed by the multiply-adds)
            float *bs = reinterpret_cast<float *>(smem + XR_WAVES * XR_STAGE + bi * XR_SUMS);
#pragma unroll
            for (int t = 0; t < XD_TOK; ++t) bs[t * 64 + l] = a0[t];
        }
    }
    __syncthreads();
    // group sums: wave w chains the block sums of tokens w, w + 4, w + 8, w + 12 in ascending order
#pragma unroll
    for (int u = 0; u < XD_TOK / XR_WAVES; ++u) {
        const int tl = w + XR_WAVES * u;
        const int t = t0 + tl;
        if (t < T) {
            float s0 = 0.f;
            for (int i = 0; i < nb; ++i) s0 = __fadd_rn(s0, reinterpret_cast<const float *>(smem + XR_WAVES * XR_STAGE + i * XR_SUMS)[tl * 64 + l]);
            sl.out[(size_t)t * sl.out_pitch + l] = s0;
        }
    }
}

}  // namespace
}  // namespace pto
