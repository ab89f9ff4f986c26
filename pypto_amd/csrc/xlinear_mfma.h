// Sums over the hidden axis on the matrix cores, for prefill-sized token counts: x [T, h] bf16 times a slab of up
// to 128 columns of a row-major bf16 weight matrix, as partial sums over a range of the hidden axis.  Shared by the
// MLA prolog (w_dq, w_dkv_kr) and the lightning-indexer prolog (wk, w_proj); included after prolog_common.h.
//
// All products are exact in fp32 (bf16 x bf16); the sums are taken in the cores' own order, so the results may
// differ from the fixed-order sums of the decode kernels in the last bit.
//   workgroup = (slab, range of the hidden axis, 128 tokens), four waves: wave (wc, wt) holds columns
//   64*wc .. +63 x tokens 64*wt .. +63 as four 32x32 accumulators of
//   O^T[column][token] = sum_k W^T[column][k] x^T[k][token]
//   A = W^T: the slab's rows are row-major [k][columns], so the operand is read from LDS with the transposing
//   ds_read_b64_tr_b16; B = x^T: lane (token, half) holds 8 consecutive hidden states of its token.
//   Chunks of 64 hidden rows travel by LDS-DMA into two buffers (16 KiB of the slab + 16 KiB of hidden states
//   each), the next chunk under the products of the current one.  16-byte piece q of slab row r sits at piece q ^ 4*(r & 3),
//   piece q of token row t at q ^ ((t >> 1) & 7): the four rows of a transposing read and the 32 token rows of an
//   operand read then spread over all banks.  A slab narrower than 128 columns (8 * pieces) is staged unswizzled
//   by the lanes whose pieces exist; the columns past its end hold whatever the buffer held and are not stored.
#pragma once
#include "prolog_common.h"

namespace pto {
namespace {

constexpr int XM_TOK = 128;                      // tokens per workgroup
constexpr int XM_KC = 64;                        // hidden rows per chunk
constexpr int XM_W_BYTES = XM_KC * 256;          // slab rows are staged 256 bytes apart
constexpr int XM_X_BYTES = XM_TOK * XM_KC * 2;
constexpr int XM_BUF = XM_W_BYTES + XM_X_BYTES;
constexpr int XM_LDS = 2 * XM_BUF;
constexpr int XM_SPITCH = 272;                   // bytes between the rows of a wave's output staging area (32 tokens x 64 columns fp32)

struct XmSlab {
    const uint8_t *w;     // column 0 of the slab in row 0 of the weight matrix
    int pitch;            // bytes between rows of the weight matrix
    int pieces;           // 16-byte pieces of a row that belong to the slab: 16, or fewer for a narrow one
    float *out;           // partial sums of this range: out[t * out_pitch + column of the slab]
    int out_pitch;
};

// chunks [c_begin, c_end) of the hidden axis, tokens t0 .. t0 + 127 (rows past T - 1 repeat it and are not stored)
__device__ __forceinline__ void xm_body(const XmSlab &sl, const uint16_t *x, const int T, const int h, const int t0, const int c_begin,
                                        const int c_end, uint8_t *smem)
{
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wc = w & 1, wt = w >> 1;
    const bool narrow = sl.pieces < 16;
    const bool idle = sl.pieces <= 8 && wc == 1;                   // no column of this wave's half exists
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_byte_t *)smem;

    // this wave's eight requests of a chunk: four of the slab (four rows each), four of the hidden states (eight
    // token rows each).  Their addresses are made once, for chunk 0; a chunk further on is a uniform number of bytes
    // further on (the loop then spends two additions per request instead of rebuilding the addresses).
    const int wrow = l >> 4, wpos = l & 15;
    const uint32_t woff = (uint32_t)(wrow * sl.pitch + 16 * (narrow ? (wpos < sl.pieces ? wpos : 0) : (wpos ^ (4 * wrow))));
    const uint64_t wmask = narrow ? ((1ull << sl.pieces) - 1) * 0x0001000100010001ull : ~0ull;
    const int xrow = l >> 3, xpos = l & 7;
    const uint8_t *wreq[4], *xreq[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int req = 4 * w + j;
        wreq[j] = sl.w + (size_t)(4 * req) * sl.pitch + woff;
        const int tl = 8 * req + xrow;                              // token row inside the workgroup's 128
        int t = t0 + tl;
        t = t < T ? t : T - 1;
        xreq[j] = reinterpret_cast<const uint8_t *>(x) + (size_t)t * h * 2 + 16 * (xpos ^ ((tl >> 1) & 7));
    }
    const size_t wstep = (size_t)XM_KC * sl.pitch;
    auto request_chunk = [&](const int c, const int buf) {
        const uint32_t dst = lds0 + (uint32_t)(buf * XM_BUF);
#pragma unroll
        for (int j = 0; j < 4; ++j) dma16_lanes(wreq[j] + (size_t)c * wstep, dst + 1024u * (4 * w + j), wmask);
#pragma unroll
        for (int j = 0; j < 4; ++j) dma16(xreq[j] + (size_t)c * (XM_KC * 2), dst + XM_W_BYTES + 1024u * (4 * w + j));
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[cb][tb][r] = 0.f;

    // per-lane read offsets inside a buffer
    // A: row 16*ks + 8*(l>>5) + (l&15)>>2 (+4), column 64*wc + 32*cb + 16*((l>>4)&1) + 4*(l&3)
    const int arow = 8 * (l >> 5) + ((l & 15) >> 2);
    const int aswz = narrow ? 0 : 4 * ((l & 15) >> 2);
    uint32_t aoff[2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
        const int piece = 8 * wc + 4 * cb + 2 * ((l >> 4) & 1) + ((l & 3) >> 1);
        aoff[cb] = (uint32_t)(arow * 256 + 16 * (piece ^ aswz) + 8 * (l & 1));
    }
    // B: token row 64*wt + 32*tb + (l&31), piece 2*ks + (l>>5)
    const int brow = 64 * wt + (l & 31);
    const int bswz = (brow >> 1) & 7;
    // the next chunk is requested into the other buffer before the current one is waited for; two workgroups share a
    // compute unit, so eight waves keep requests in flight (the rate of LDS-DMA grows with the waves that issue it)
    if (c_begin < c_end) request_chunk(c_begin, 0);
    int buf = 0;
#pragma unroll 1
    for (int c = c_begin; c < c_end; ++c) {
        if (c + 1 < c_end) {
            request_chunk(c + 1, buf ^ 1);
            VM_WAIT(8);
        } else {
            VM_WAIT(0);
        }
        __syncthreads();                                           // every wave's part of chunk c has landed
        const uint8_t *wb = smem + buf * XM_BUF;
        const uint8_t *xb = wb + XM_W_BYTES;
        if (!idle) {
#pragma unroll
            for (int ks = 0; ks < XM_KC / 16; ++ks) {
                bf16x8 a[2], b[2];
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) {
                    const uint16_t *ap = reinterpret_cast<const uint16_t *>(wb + aoff[cb] + 16 * ks * 256);
                    const s16x4 lo = lds_read_tr16(ap), hi = lds_read_tr16(ap + 4 * 128);
                    a[cb] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
#pragma unroll
                for (int tb = 0; tb < 2; ++tb)
                    b[tb] = *reinterpret_cast<const bf16x8 *>(xb + (brow + 32 * tb) * 128 + 16 * ((2 * ks + (l >> 5)) ^ bswz));
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                    for (int tb = 0; tb < 2; ++tb)
                        acc[cb][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[cb], b[tb], acc[cb][tb], 0, 0, 0);
            }
        }
        buf ^= 1;
        __syncthreads();                                           // the buffer may be requested into again
    }
    // accumulator register r of lane (token, half) is column 8*(r/4) + 4*half + r%4 of its 32-column block: 16-byte
    // fragments of 32 different rows per store; they leave through a staging area of the wave's own (the chunk
    // buffers are free past the loop's last barrier) as whole 256-byte row segments instead
    static_assert(4 * 32 * XM_SPITCH <= XM_LDS, "the staging areas reuse the chunk buffers");
    if (!idle) {
        uint8_t *stg = smem + w * (32 * XM_SPITCH);
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
            uint8_t *row = stg + (l & 31) * XM_SPITCH + 16 * (l >> 5);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 v = {acc[cb][tb][4 * q], acc[cb][tb][4 * q + 1], acc[cb][tb][4 * q + 2], acc[cb][tb][4 * q + 3]};
                    *reinterpret_cast<f32x4 *>(row + 128 * cb + 32 * q) = v;
                }
            // the wave reads back what it wrote itself: LDS operations of a wave stay in order
            const int col = 64 * wc + 4 * (l & 15);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int r = 4 * k + (l >> 4);
                const f32x4 v = *reinterpret_cast<const f32x4 *>(stg + r * XM_SPITCH + 16 * (l & 15));
                const int t = t0 + 64 * wt + 32 * tb + r;
                if (t < T && col < 8 * sl.pieces) *reinterpret_cast<f32x4 *>(sl.out + (size_t)t * sl.out_pitch + col) = v;
            }
        }
    }
}

}  // namespace
}  // namespace pto
