// Device helpers shared by the two prolog kernels files (lightning-indexer prolog, MLA prolog):
// explicit vector-memory waits, the int8 projection job (row-major int8 weight tile -> LDS by LDS-DMA
// -> v_mfma_i32_32x32x32_i8), fp32 wave reductions in a fixed order without LDS traffic.
#pragma once
#include "common.h"

namespace pto {
namespace {

constexpr int QPROJ_KSPLIT = 4;     // jobs that share the reduction axis of the int8 projection
constexpr int QPROJ_PREFILL_TOKENS = 64;   // from this many tokens on the projection runs unsplit (q_prefill_body)

// partial sums per output of the int8 projection at T tokens
__host__ __device__ inline int qproj_splits(const int T) { return T >= QPROJ_PREFILL_TOKENS ? 1 : QPROJ_KSPLIT; }

struct QProj {
    const int8_t *q_norm;   // [T, q_lora]
    const int8_t *w;        // [q_lora, 128 * nslabs], row-major
    int32_t *part;          // split form: int32 partial sums [QPROJ_KSPLIT, T, 128 * nslabs]; unsplit form: the
                            // de-quantised results as bf16 [T, 128 * nslabs] (half the bytes on their way to the
                            // last launch, which would de-quantise them first thing anyway)
    int T, q_lora, nslabs;
    const float *tok_scale; // [T]              } result = bf16((float(sum) * tok_scale[t]) * col_scale[column]),
    const float *col_scale; // [128 * nslabs]   } read by the unsplit form only
};

#define VM_WAIT(n) __builtin_amdgcn_s_waitcnt((((n) & 15) | (((n) >> 4) << 14) | 0x0F70))

// at most n (a multiple of 4, <= 60) vector-memory requests of this wave still outstanding
__device__ __forceinline__ void wait_vm_le(const int n)
{
    switch (n) {
    case 4: VM_WAIT(4); break;
    case 8: VM_WAIT(8); break;
    case 12: VM_WAIT(12); break;
    case 16: VM_WAIT(16); break;
    case 20: VM_WAIT(20); break;
    case 24: VM_WAIT(24); break;
    case 28: VM_WAIT(28); break;
    case 32: VM_WAIT(32); break;
    case 36: VM_WAIT(36); break;
    case 40: VM_WAIT(40); break;
    case 44: VM_WAIT(44); break;
    default: VM_WAIT(0); break;
    }
}

__device__ __forceinline__ float bf16_round_f32(const float v)
{
    return __uint_as_float(pack_bf16x2(v, 0.0f) << 16);
}

// Weight operands by the transposing 8-bit LDS read.  ds_read_b64_tr_b8 takes, per group of
// 16 lanes, the 16 rows of 8 bytes its lanes point at and hands lane j byte j of the even lanes' rows and lane 8 + j
// byte j of the odd lanes' rows.  Even lanes point at eight consecutive rows of the tile at one block of 8 columns,
// odd lanes at the same rows of the next block: lane n of the group then holds column n of 16, eight rows deep --
// half of what v_mfma_i32_32x32x32_i8 wants from a lane (column l % 32, rows 16*(l / 32) .. +15), so two reads per
// product and no byte shuffling.  Product i covers columns 32*i .. 32*i + 31 of the slab.
// Tile layout the reads assume: row r (128 bytes) keeps its 16-byte piece q at piece q ^ 2*((r >> 1) & 3), so that
// the eight rows of a half-wave's read fall on different banks; the LDS-DMA requests place the pieces that way.
__device__ __forceinline__ int q_tr_piece_swizzle(const int row) { return 2 * ((row >> 1) & 3); }

// the operand of product i alone
__device__ __forceinline__ i32x4 q_build_a_tr_one(const uint8_t *tile, const int s, const int l, const int i)
{
    typedef int v2i __attribute__((ext_vector_type(2)));
    const int x = (l >> 2) & 3;
    const uint8_t *pi = tile + (32 * s + 16 * (l >> 5) + ((l & 15) >> 1)) * 128 + 16 * ((l >> 4) & 1) + 8 * (l & 1) + 32 * (i ^ x);
    const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(lds_byte_t *)pi);
    const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(lds_byte_t *)(pi + 8 * 128));
    const i32x4 a = {lo[0], lo[1], hi[0], hi[1]};
    return a;
}

__device__ __forceinline__ void q_build_a_tr(const uint8_t *tile, const int s, const int l, i32x4 (&a)[4])
{
    typedef int v2i __attribute__((ext_vector_type(2)));
    const int x = (l >> 2) & 3;                         // (row >> 1) & 3 of this lane's rows
    const uint8_t *base = tile + (32 * s + 16 * (l >> 5) + ((l & 15) >> 1)) * 128 + 16 * ((l >> 4) & 1) + 8 * (l & 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint8_t *pi = base + 32 * (i ^ x);
        const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(lds_byte_t *)pi);
        const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(lds_byte_t *)(pi + 8 * 128));
        a[i][0] = lo[0];
        a[i][1] = lo[1];
        a[i][2] = hi[0];
        a[i][3] = hi[1];
    }
}

// ---------------------------------------------------------------------------------------------
// Int8 projection [T, q_lora] x [q_lora, 128*nslabs] -> partial int32 sums: one job per (slab of 128 columns, quarter of the reduction axis, block of 32 tokens); its
// waves 0 and 1 take one half of the quarter each (HS steps of 32 rows).
// LDS region of a wave: [tile: 32*HS rows x 128 bytes][token operands: HS x 1024 bytes].
// Matrix product per step: A = 32 output columns x 32 rows of the tile (product i: columns 32i .. 32i+31; lane l
// holds rows 16*(l/32) .. +15 of column 32i + l%32, q_build_a_tr), B = 32 tokens x the same 32 rows of q_norm, so
// that accumulator registers 4*rg .. 4*rg+3 of product i hold columns 32i + 8*rg + 4*(l/32) .. +3 of token l%32.
template <int HS>
__device__ __forceinline__ void q_issue(const QProj &p, uint8_t *region, const int job, const int half)
{
    const int l = threadIdx.x & 63;
    const int ncols = p.nslabs * 128;
    const int kq = job & (QPROJ_KSPLIT - 1);
    const int head = (job >> 2) % p.nslabs;
    const int tb = (job >> 2) / p.nslabs;
    constexpr int KH = HS * 32;                        // rows of this wave
    constexpr int NW = KH / 8;                         // tile requests of 8 rows each
    const int k0 = (kq * 2 + half) * KH;
    const uint32_t tile = (uint32_t)(uintptr_t)(lds_byte_t *)region;
    const uint32_t tok = tile + KH * 128;

    // token operands and the tile: every request is issued before the first wait.  The loops stay
    // rolled: straight-line code that runs once is bound by instruction fetch.
    {
        int t = tb * 32 + (l & 31);
        t = t < p.T ? t : p.T - 1;
        const int8_t *src = p.q_norm + (size_t)t * p.q_lora + k0 + 16 * (l >> 5);
#pragma unroll 1
        for (int s = 0; s < HS; ++s) dma16(src + 32 * s, tok + 1024 * s);
    }
    {   // lane l fills piece l % 8 of row l / 8 of a request's eight rows, with the piece q_build_a_tr expects there
        const int8_t *src = p.w + ((size_t)k0 + (l >> 3)) * ncols + head * 128 + 16 * ((l & 7) ^ q_tr_piece_swizzle(l >> 3));
#pragma unroll 1
        for (int i = 0; i < NW; i += 4) {
            dma16(src + (size_t)i * 8 * ncols, tile + 1024 * i);
            dma16(src + (size_t)(i + 1) * 8 * ncols, tile + 1024 * (i + 1));
            dma16(src + (size_t)(i + 2) * 8 * ncols, tile + 1024 * (i + 2));
            dma16(src + (size_t)(i + 3) * 8 * ncols, tile + 1024 * (i + 3));
        }
    }
}

// one 32-row step of the product: rows 32s.. of the tile, token operands of step s at tok + 1024 s
__device__ __forceinline__ void q_step_at(const uint8_t *tile, const uint8_t *tok, const int s, const int l, i32x16 (&acc)[4])
{
    i32x4 a[4];
    q_build_a_tr(tile, s, l, a);
    const i32x4 b = *reinterpret_cast<const i32x4 *>(tok + 1024 * s + 16 * l);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b, acc[i], 0, 0, 0);
}
// the same from a wave's region of a split job
template <int HS>
__device__ __forceinline__ void q_step(const uint8_t *region, const int s, const int l, i32x16 (&acc)[4])
{
    q_step_at(region, region + HS * 32 * 128, s, l, acc);
}

// A single job: issue, then every step as soon as its four requests have landed (requests complete
// in order), so only the last step trails the arrival of the tile.
template <int HS>
__device__ __forceinline__ void q_half_job(const QProj &p, uint8_t *region, const int job, const int half, i32x16 (&acc)[4])
{
    constexpr int NW = HS * 4;
    q_issue<HS>(p, region, job, half);
    const int l = threadIdx.x & 63;
#pragma unroll
    for (int s = 0; s < HS; ++s) {
        wait_vm_le(NW - 4 * (s + 1));
        q_step<HS>(region, s, l, acc);
    }
}

constexpr int LIN_RED_BYTES = 16 * 64 * 16;           // one wave's accumulators, 16 bytes per (register, lane)

template <int HS>
constexpr int lin_region_bytes()
{
    return HS * (32 * 128 + 1024) > LIN_RED_BYTES ? HS * (32 * 128 + 1024) : LIN_RED_BYTES;
}

// Both halves done (the caller has passed a workgroup barrier since wave 1 parked its accumulators at
// `parked`): wave 0 adds them to its own and stores the partial sums of its 32 tokens x 128 columns.
__device__ __forceinline__ void q_pair_store_from(const QProj &p, const uint8_t *parked, const int job, const int l, const i32x16 (&acc)[4])
{
    const i32x4 *red = reinterpret_cast<const i32x4 *>(parked);
    const int ncols = p.nslabs * 128;
    const int kq = job & (QPROJ_KSPLIT - 1);
    const int head = (job >> 2) % p.nslabs;
    const int t = ((job >> 2) / p.nslabs) * 32 + (l & 31);
    if (t < p.T) {
        int32_t *dst = p.part + ((size_t)kq * p.T + t) * ncols + head * 128;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const i32x4 o = red[(4 * i + rg) * 64 + l];
                i32x4 v = {acc[i][4 * rg] + o[0], acc[i][4 * rg + 1] + o[1], acc[i][4 * rg + 2] + o[2], acc[i][4 * rg + 3] + o[3]};
                *reinterpret_cast<i32x4 *>(dst + 32 * i + 8 * rg + 4 * (l >> 5)) = v;
            }
    }
}
// the same with wave 1's accumulators parked in its own (consumed) tile region, the second of two
template <int HS>
__device__ __forceinline__ void q_pair_store(const QProj &p, const uint8_t *smem, const int job, const int l, const i32x16 (&acc)[4])
{
    q_pair_store_from(p, smem + lin_region_bytes<HS>(), job, l, acc);
}
// wave 1 parks its accumulators in its own (consumed) tile region
__device__ __forceinline__ void q_pair_park(uint8_t *region, const int l, const i32x16 (&acc)[4])
{
    i32x4 *red = reinterpret_cast<i32x4 *>(region);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            i32x4 v = {acc[i][4 * rg], acc[i][4 * rg + 1], acc[i][4 * rg + 2], acc[i][4 * rg + 3]};
            red[(4 * i + rg) * 64 + l] = v;
        }
}

// The unsplit forms' results leave de-quantised, as bf16, through a staging area of the wave's own in LDS
// (Q_STAGE_BYTES; the chunk buffers are free by then), so that they reach memory as whole 256-byte rows instead of
// 8-byte fragments of 32 different rows: registers 4*rg .. 4*rg+3 of product i hold columns 32*i + 8*rg + 4*(l/32) .. +3
// of this lane's token (q_build_a_tr).  tbase: first of the wave's 32 tokens; col0: first of its 128 columns.
constexpr int Q_STAGE_PITCH = 272;                     // bytes between token rows: 16-byte aligned, 4 banks apart
constexpr int Q_STAGE_BYTES = 32 * Q_STAGE_PITCH;
// products i0 .. i0+NP-1 of a wave (columns 32*i0 .. of the 128 at col0) go to the staging area of their token block
template <int NP>
__device__ __forceinline__ void q_stage_products(const QProj &p, const i32x16 (&acc)[NP], const int i0, const int tbase, const int col0, const int l,
                                                 uint8_t *stage)
{
    const int t = tbase + (l & 31);
    const float ts = p.tok_scale[t < p.T ? t : p.T - 1];
    const float *cs = p.col_scale + col0;
    uint8_t *mine = stage + (l & 31) * Q_STAGE_PITCH;
#pragma unroll
    for (int i = 0; i < NP; ++i)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            const int col = 32 * (i0 + i) + 8 * rg + 4 * (l >> 5);
            const f32x4 c = *reinterpret_cast<const f32x4 *>(cs + col);
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = __fmul_rn(__fmul_rn((float)acc[i][4 * rg + j], ts), c[j]);
            const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2 *>(mine + 2 * col) = o;
        }
}
// rows 4*k .. 4*k+3 (k = k_begin .. k_end-1) of a staged token block leave as whole 256-byte rows
__device__ __forceinline__ void q_store_rows(const QProj &p, const int tbase, const int col0, const int l, const uint8_t *stage, const int k_begin,
                                             const int k_end)
{
    const int ncols = p.nslabs * 128;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.part) + col0 + 8 * (l & 15);
#pragma unroll
    for (int k = k_begin; k < k_end; ++k) {
        const int row = 4 * k + (l >> 4);
        const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + row * Q_STAGE_PITCH + 16 * (l & 15));
        if (tbase + row < p.T) *reinterpret_cast<u32x4 *>(dst + (size_t)(tbase + row) * ncols) = v;
    }
}
__device__ __forceinline__ void q_store_dequantised(const QProj &p, const i32x16 (&acc)[4], const int tbase, const int col0, const int l,
                                                    uint8_t *stage)
{
    q_stage_products<4>(p, acc, 0, tbase, col0, l, stage);
    // the wave reads back what it wrote itself: LDS operations of a wave stay in order
    q_store_rows(p, tbase, col0, l, stage, 0, 8);
}

// ---------------------------------------------------------------------------------------------
// The projection at prefill sizes (T >= QPROJ_PREFILL_TOKENS): one workgroup of four waves per (slab of 128
// columns, block of 128 tokens) walks the whole reduction axis in chunks of 128 rows, so a weight tile is read
// once per 128 tokens instead of once per 32 and no partial sums are left to add.  Wave w takes tokens 32w..32w+31
// of the block; the chunk of the tile (16 KiB, shared) and each wave's token operands (4 KiB) travel by LDS-DMA into
// one of two buffers, a chunk ahead of the products that read them.  Same products as a split job; the weight
// operands come out of LDS by the transposing 8-bit read (q_build_a_tr) instead of byte shuffles.
constexpr int QPF_STEPS = 4;                           // 32-row steps per chunk
constexpr int QPF_TILE = QPF_STEPS * 32 * 128;
constexpr int QPF_TOK = QPF_STEPS * 1024;
constexpr int QPF_BUF = QPF_TILE + 4 * QPF_TOK;
constexpr int QPF_LDS = 2 * QPF_BUF;                   // 64 KiB

__host__ __device__ inline int q_prefill_jobs(const QProj &p) { return p.nslabs * ((p.T + 127) / 128); }
// token blocks per tile of the form to take: a launch of one tile of one or two blocks has forms of its own
__host__ __device__ inline int q_prefill_token_blocks(const int T) { return T <= 32 ? 1 : (T <= 64 ? 2 : 4); }

// job: the blocks of a slab are neighbours in the job order.
// TB: blocks of 32 tokens the tile holds.  TB = 4 is the form described above.  A launch of at most 32 or 64 tokens
// (one tile of TB = 1 or 2 blocks per slab) shares a token block among 4 / TB waves, each with TB of the four
// 32-column products: a wave then issues 4 or 8 products per chunk instead of 16 on padding tokens, and the
// kernel's time is its requests' and no longer a wave's products'.  Same integer sums, same conversion.
template <int TB = 4>
__device__ __forceinline__ void q_prefill_body(const QProj &p, const int job, uint8_t *lds)
{
    static_assert(TB == 1 || TB == 2 || TB == 4, "token blocks per tile");
    constexpr int WPB = 4 / TB;                        // waves that share a token block
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tb = w % TB;                             // this wave's token block
    const int i0 = (w / TB) * TB;                      // its first product (32 columns each)
    const int ncols = p.nslabs * 128;
    const int ttiles = (p.T + 32 * TB - 1) / (32 * TB);
    const int slab = job / ttiles;
    const int tile0 = (job % ttiles) * (32 * TB);
    const int nch = p.q_lora / (32 * QPF_STEPS);
    // token operands: a request brings 128 bytes (the chunk's four steps) of 8 tokens -- whole lines; as 32 tokens x 32
    // bytes a request runs at half the rate.  Lane l fills piece l % 8 of token row l / 8 with piece (l % 8) ^ (l / 8)
    // of that token, so that the operand reads of 8 consecutive tokens fall on different banks.  The four requests
    // of a token block are dealt to the waves that share it.
    const int8_t *tsrc[TB];
    int treq[TB];
#pragma unroll
    for (int k = 0; k < TB; ++k) {
        const int i = (w / TB) + WPB * k;              // request (eight tokens) of block tb
        treq[k] = i;
        int tq = tile0 + 32 * tb + 8 * i + (l >> 3);
        tq = tq < p.T ? tq : p.T - 1;                  // rows past the end repeat the last token and are not stored
        tsrc[k] = p.q_norm + (size_t)tq * p.q_lora + 16 * ((l & 7) ^ (l >> 3));
    }
    // lane l of a tile request fills piece l % 8 of row l / 8 of its eight rows: with the piece that belongs there (q_build_a_tr)
    const int8_t *wsrc = p.w + (size_t)(32 * w + (l >> 3)) * ncols + slab * 128 + 16 * ((l & 7) ^ q_tr_piece_swizzle(l >> 3));
    const uint32_t base = (uint32_t)(uintptr_t)(lds_byte_t *)lds;
    auto issue = [&](const int c, const int b) {
        const uint32_t buf = base + b * QPF_BUF;
#pragma unroll
        for (int k = 0; k < TB; ++k) dma16(tsrc[k] + c * (32 * QPF_STEPS), buf + QPF_TILE + tb * QPF_TOK + 1024 * treq[k]);
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(wsrc + ((size_t)c * (32 * QPF_STEPS) + 8 * i) * ncols, buf + 1024 * (4 * w + i));
    };
    i32x16 acc[TB];
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    auto products = [&](const uint8_t *buf) {
#pragma unroll
        for (int s = 0; s < QPF_STEPS; ++s) {
            const i32x4 b = *reinterpret_cast<const i32x4 *>(buf + QPF_TILE + tb * QPF_TOK + (l & 31) * 128 + 16 * ((2 * s + (l >> 5)) ^ (l & 7)));
            if (TB == 4) {
                i32x4 a[4];
                q_build_a_tr(buf, s, l, a);
#pragma unroll
                for (int i = 0; i < TB; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b, acc[i], 0, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < TB; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q_build_a_tr_one(buf, s, l, i0 + i), b, acc[i], 0, 0, 0);
            }
        }
    };
    constexpr int PER_CHUNK = TB + 4;                  // a wave's requests of a chunk
    issue(0, 0);
#pragma unroll 1
    for (int c = 0; c < nch; ++c) {
        if (c + 1 < nch) {
            issue(c + 1, (c + 1) & 1);
            VM_WAIT(PER_CHUNK);
        } else {
            VM_WAIT(0);
        }
        __syncthreads();                               // every wave's share of chunk c has landed
        products(lds + (c & 1) * QPF_BUF);
        __syncthreads();                               // chunk c + 2 goes where chunk c was read
    }
    static_assert(4 * Q_STAGE_BYTES <= QPF_LDS, "the staging areas reuse the chunk buffers");
    // past the loop's last barrier: every token block has a staging area, filled by the waves that share the block
    uint8_t *stage = lds + tb * Q_STAGE_BYTES;
    q_stage_products<TB>(p, acc, i0, tile0 + 32 * tb, slab * 128, l, stage);
    if (TB < 4) __syncthreads();                       // (a wave of the TB = 4 form reads back only what it wrote itself)
    q_store_rows(p, tile0 + 32 * tb, slab * 128, l, stage, (w / TB) * 2 * TB, (w / TB + 1) * 2 * TB);
}
// The same projection for grids that fill the chip with larger tiles: a workgroup of eight waves per (256 columns,
// 256 tokens); wave (wc, wt) holds columns 128*wc .. +127 x tokens 64*wt .. +63 (eight accumulators), so a weight
// operand built from LDS serves two token blocks and every byte staged serves four times the products of the
// 128 x 128 form -- these kernels are bound by the operand traffic from the L2 into LDS, not by the matrix cores.
// Chunks of 64 rows (two steps): the tile as two halves of [64 rows][128 bytes] and the token operands of eight
// token blocks x two steps, 32 KiB, in three buffers two chunks ahead of the products; one barrier per chunk.
constexpr int QP2_BUF = 2 * 64 * 128 + 16 * 1024;
constexpr int QP2_NBUF = 3;
constexpr int QP2_LDS = QP2_NBUF * QP2_BUF;            // 96 KiB

__host__ __device__ inline int q_prefill256_jobs(const QProj &p) { return ((p.nslabs + 1) / 2) * ((p.T + 255) / 256); }

__device__ __forceinline__ void q_prefill256_body(const QProj &p, const int job, uint8_t *lds)
{
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wc = w & 1, wt = w >> 1;
    const int ncols = p.nslabs * 128;
    const int ttiles = (p.T + 255) / 256;
    const int ct = job / ttiles;
    const int t0 = (job % ttiles) * 256;
    const int nch = p.q_lora / 64;
    const bool cols_live = 2 * ct + wc < p.nslabs;      // an odd number of slabs leaves the last tile half empty
    const uint32_t base = (uint32_t)(uintptr_t)(lds_byte_t *)lds;
    // this wave's four requests of a chunk: tile pieces 2w, 2w+1 (half = piece / 8; rows 8*(piece % 8) .. +7 of the
    // chunk, 16-byte pieces placed as q_build_a_tr reads them) and token pieces 2w, 2w+1 (token block w, steps 0 and 1)
    const int8_t *tsrc[2];
    uint32_t tdst[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int q = 2 * w + j;
        const int half = q >> 3, rb = q & 7;
        const int slab = 2 * ct + half < p.nslabs ? 2 * ct + half : p.nslabs - 1;
        tsrc[j] = p.w + (size_t)(8 * rb + (l >> 3)) * ncols + slab * 128 + 16 * ((l & 7) ^ q_tr_piece_swizzle(l >> 3));
        tdst[j] = half * 8192 + rb * 1024;
    }
    int t = t0 + 32 * w + (l & 31);
    t = t < p.T ? t : p.T - 1;
    const int8_t *ksrc = p.q_norm + (size_t)t * p.q_lora + 16 * (l >> 5);
    auto issue = [&](const int c, const int buf) {
        const uint32_t b = base + buf * QP2_BUF;
#pragma unroll
        for (int j = 0; j < 2; ++j) dma16(tsrc[j] + (size_t)c * 64 * ncols, b + tdst[j]);
#pragma unroll
        for (int s = 0; s < 2; ++s) dma16(ksrc + c * 64 + 32 * s, b + 16384 + (2 * w + s) * 1024);
    };
    i32x16 acc[2][4];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tb][i][r] = 0;
    issue(0, 0);
    if (nch > 1) issue(1, 1);
    int buf = 0;
#pragma unroll 1
    for (int c = 0; c < nch; ++c) {
        if (c + 1 < nch) VM_WAIT(4);
        else VM_WAIT(0);
        __syncthreads();                               // chunk c has landed for every wave; every wave is done with chunk c - 1
        if (c + 2 < nch) issue(c + 2, buf == 0 ? 2 : buf - 1);
        const uint8_t *bp = lds + buf * QP2_BUF;
        if (cols_live) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                i32x4 a[4];
                q_build_a_tr(bp + wc * 8192, s, l, a);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    const i32x4 b = *reinterpret_cast<const i32x4 *>(bp + 16384 + (2 * (2 * wt + tb) + s) * 1024 + 16 * l);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[tb][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b, acc[tb][i], 0, 0, 0);
                }
            }
        }
        buf = buf == 2 ? 0 : buf + 1;
    }
    static_assert(8 * Q_STAGE_BYTES <= QP2_LDS, "the staging areas reuse the chunk buffers");
    __syncthreads();                                   // every wave is done with the last chunk
    if (cols_live) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) q_store_dequantised(p, acc[tb], t0 + 64 * wt + 32 * tb, (2 * ct + wc) * 128, l, lds + w * Q_STAGE_BYTES);
    }
}

// workgroup number -> job, so that the workgroups of a slab (consecutive jobs) run on one XCD (workgroups go round
// the eight XCDs) and share its L2 copy of the weight tile
__device__ __forceinline__ int q_prefill_job_of(const int wg, const int njobs)
{
    return (njobs & 7) == 0 ? (wg & 7) * (njobs >> 3) + (wg >> 3) : wg;
}

// Cross-lane exchanges without LDS traffic.  dpp_f32 reads another lane of the same row of 16;
// row_swap16 / half_swap32 return {own-side, other-side} copies across rows of 16 / halves of 32
// (v_permlane16_swap, v_permlane32_swap with both operands equal).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(const float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
constexpr int DPP_XOR1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141;  // lane i of a group of 8 reads lane 7-i
constexpr int DPP_MIRROR = 0x140;     // lane i of a row of 16 reads lane 15-i

// value held by lane l ^ 16
__device__ __forceinline__ float xor16_f32(const float v, const int l)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    // r[0]: rows 0,0,2,2 of v;  r[1]: rows 1,1,3,3
    return __uint_as_float((l & 16) ? r[0] : r[1]);
}

// combine(own, partner) over the whole wave where combine is commutative and every step leaves all
// lanes of the finished group with the same bits: xor 1, xor 2, then mirrors within 8 and 16 lanes
// (the mirrored lane lies in the other half, which is uniform), then the row and half swaps.
#define WAVE_BUTTERFLY(v, OP)                                                                              \
    do {                                                                                                   \
        v = OP(v, dpp_f32<DPP_XOR1>(v));                                                                   \
        v = OP(v, dpp_f32<DPP_XOR2>(v));                                                                   \
        v = OP(v, dpp_f32<DPP_HALF_MIRROR>(v));                                                            \
        v = OP(v, dpp_f32<DPP_MIRROR>(v));                                                                 \
        {                                                                                                  \
            const auto r_ = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false); \
            v = OP(__uint_as_float(r_[0]), __uint_as_float(r_[1]));                                        \
        }                                                                                                  \
        {                                                                                                  \
            const auto r_ = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false); \
            v = OP(__uint_as_float(r_[0]), __uint_as_float(r_[1]));                                        \
        }                                                                                                  \
    } while (0)

__device__ __forceinline__ float wave_max_f32(float v)
{
    WAVE_BUTTERFLY(v, fmaxf);
    return v;
}

// sum of the wave's 128 values (two per lane, neighbours) as a balanced tree over neighbours
__device__ __forceinline__ float pair_tree_sum(const float v0, const float v1)
{
    float s = __fadd_rn(v0, v1);
    WAVE_BUTTERFLY(s, __fadd_rn);
    return s;
}


// symmetric int8 quantisation of two values per lane against a given maximum of magnitudes; returns
// the packed byte pair and the de-quantisation scale (both 0 when the maximum is 0)
__device__ __forceinline__ uint16_t quant_pair_amax(const float y0, const float y1, const float amax, float &deq)
{
    if (amax > 0.f) {
        const float s = __fdiv_rn(127.0f, amax);
        const int q0 = (int)rintf(__fmul_rn(y0, s));
        const int q1 = (int)rintf(__fmul_rn(y1, s));
        deq = __fdiv_rn(1.0f, s);
        return (uint16_t)((q0 & 0xff) | ((q1 & 0xff) << 8));
    }
    deq = 0.f;
    return 0;
}

}  // namespace
}  // namespace pto
