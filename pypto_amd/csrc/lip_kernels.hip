// Lightning-indexer prolog for gfx950: projects a decode batch of hidden states into the indexer's
// int8 query heads, its int8 key row (scattered into the paged key cache) and its per-head weights.
//
// Arithmetic (reference golden: examples/models/deepseek_v32_exp/
// deepseekv32_lightning_indexer_prolog_quant.py:216-281; operator graph:
// examples/models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:325-504):
//   query   int8 x int8 -> int32 projection, exact; * q_norm_scale * w_qb_scale in fp32; -> bf16;
//           rope on channels 0..63; 128x128 "Hadamard" product; per-(token, head) int8 quantisation
//   key     x . wk in fp32; layer norm; -> bf16; rope; Hadamard; int8 quantisation; scatter
//   weights bf16(x . w_proj) * n_heads^-1/2 * 128^-1/2 -> fp16
// Every product of two bf16 values is exact in fp32, so each fp32 sum is fixed by its order alone.
// The orders used here: sums over the hidden axis are cut into blocks of 64 (a block ascending from
// 0.0), eight consecutive block sums are added ascending into a group sum, group sums are added
// ascending; the Hadamard sums run over i ascending; the two layer-norm means
// are balanced binary trees over neighbouring channels.  No matrix-core instruction touches these
// sums (its internal order is not specified); only the exact integer projection uses one.
//
// Two launches:
//   lip_linear_kernel   one wave per job.  Query jobs (head, quarter of the reduction axis, block of
//                       32 tokens): the quarter tile of w_qb (q_lora/4 rows x 128 bytes) and the
//                       token rows travel to LDS by LDS-DMA, all requests issued up front; each
//                       32-row step is consumed as soon as its requests have landed (they complete in
//                       order): 4x4 byte transposes (v_perm_b32) turn the row-major tile into
//                       v_mfma_i32_32x32x32_i8 operands.  Partial int32 sums go to the workspace.
//                       Hidden-axis jobs (block of 64 rows of wk and w_proj, 4 tokens): fp32 FMAs with
//                       the hidden states as scalar operands; block sums go to the workspace.
//   lip_finish_kernel   Query rows, one per wave: add the four partial sums, de-quantise, rope,
//                       Hadamard (matrix staged in LDS once per workgroup), quantise, store.  Tokens,
//                       one workgroup each: waves add the groups of block sums, then one wave finishes
//                       the key row (layer norm, rope, Hadamard, quantise, scatter) and one the weights.
#include "lip_kernels.h"
#include "common.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

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

// rows d0..d3 of four bytes each -> columns o0..o3 (o_i = byte i of d0, d1, d2, d3)
__device__ __forceinline__ void transpose4x4(const uint32_t d0, const uint32_t d1, const uint32_t d2, const uint32_t d3,
                                             uint32_t &o0, uint32_t &o1, uint32_t &o2, uint32_t &o3)
{
    const uint32_t t0 = __builtin_amdgcn_perm(d1, d0, 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(d1, d0, 0x07030602u);
    const uint32_t u0 = __builtin_amdgcn_perm(d3, d2, 0x05010400u);
    const uint32_t u1 = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
    o0 = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
    o1 = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
    o2 = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
    o3 = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
}

__device__ __forceinline__ float bf16_round_f32(const float v)
{
    return __uint_as_float(pack_bf16x2(v, 0.0f) << 16);
}

// ---------------------------------------------------------------------------------------------
// Query projection job.  STEPS = q_lora / 4 / 32 steps of 32 reduction rows.
// LDS: [tile: 32*STEPS rows x 128 bytes][token operands: STEPS x 1024 bytes].
// Matrix product per step: A = 32 output columns x 32 rows of the tile (lane (j, g) holds rows
// 16g..16g+15 of column 4j+i for product i), B = 32 tokens x the same 32 rows of q_norm, so that
// accumulator register r of lane l holds column 4*(8*(r/4) + 4*(l/32) + r%4) + i, token l%32.
template <int STEPS>
__device__ __forceinline__ void q_linear_job(const LipParams &p, uint8_t *smem, const int job)
{
    const int l = threadIdx.x;
    const int ncols = p.n_heads * LIP_DIM;
    const int kq = job & (LIP_KSPLIT - 1);
    const int head = (job >> 2) % p.n_heads;
    const int tb = (job >> 2) / p.n_heads;
    constexpr int KPER = STEPS * 32;
    constexpr int NW = KPER / 8;                       // tile requests of 8 rows each
    const uint32_t tile = (uint32_t)(uintptr_t)(lds_byte_t *)smem;
    const uint32_t tok = tile + KPER * 128;

    // token operands first (they complete first), then the tile
    {
        int t = tb * 32 + (l & 31);
        t = t < p.T ? t : p.T - 1;
        const int8_t *src = p.q_norm + (size_t)t * p.q_lora + kq * KPER + 16 * (l >> 5);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) dma16(src + 32 * s, tok + 1024 * s);
    }
    {
        const int8_t *src = p.w_qb + ((size_t)kq * KPER + (l >> 3)) * ncols + head * LIP_DIM + 16 * (l & 7);
#pragma unroll
        for (int i = 0; i < NW; ++i) dma16(src + (size_t)i * 8 * ncols, tile + 1024 * i);
    }

    i32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;

    const uint32_t *tile32 = reinterpret_cast<const uint32_t *>(smem);
    const int rd = (16 * (l >> 5)) * 32 + (l & 31);     // dword index of this lane's first row of a step
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        wait_vm_le(NW - 4 * (s + 1));
        uint32_t d[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) d[r] = tile32[s * 32 * 32 + rd + r * 32];
        const i32x4 b = *reinterpret_cast<const i32x4 *>(smem + KPER * 128 + 1024 * s + 16 * l);
        i32x4 a[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t o0, o1, o2, o3;
            transpose4x4(d[4 * q], d[4 * q + 1], d[4 * q + 2], d[4 * q + 3], o0, o1, o2, o3);
            a[0][q] = (int)o0;
            a[1][q] = (int)o1;
            a[2][q] = (int)o2;
            a[3][q] = (int)o3;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b, acc[i], 0, 0, 0);
    }

    const int t = tb * 32 + (l & 31);
    if (t < p.T) {
        int32_t *dst = p.qpart + ((size_t)kq * p.T + t) * ncols + head * LIP_DIM;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = 8 * (r >> 2) + 4 * (l >> 5) + (r & 3);
            i32x4 v = {acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
            *reinterpret_cast<i32x4 *>(dst + 4 * m) = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Hidden-axis job: block c of 64 rows of wk (lane l: columns 2l, 2l+1) and w_proj (lane l: column l),
// tokens t0..t0+3.  The hidden states are wave-uniform and are read through the scalar path.
__device__ __forceinline__ void x_linear_job(const LipParams &p, const int job)
{
    const int l = threadIdx.x;
    const int nblk = p.h / LIP_XBLOCK;
    const int c = job % nblk;
    const int t0 = (job / nblk) * 4;
    const int k0 = c * LIP_XBLOCK;
    const uint32_t *wk32 = reinterpret_cast<const uint32_t *>(p.wk) + (size_t)k0 * 64 + l;
    const bool pl = l < p.n_heads;
    const uint16_t *wp = p.w_proj + (size_t)k0 * p.n_heads + (pl ? l : 0);
    const uint32_t *xr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int tt = t0 + t < p.T ? t0 + t : p.T - 1;
        xr[t] = reinterpret_cast<const uint32_t *>(p.x + (size_t)tt * p.h + k0);
    }
    // the whole block of weights is requested before the first use
    uint32_t wv[LIP_XBLOCK];
    uint16_t pv[LIP_XBLOCK];
#pragma unroll
    for (int kk = 0; kk < LIP_XBLOCK; ++kk) wv[kk] = wk32[(size_t)kk * 64];
#pragma unroll
    for (int kk = 0; kk < LIP_XBLOCK; ++kk) pv[kk] = wp[(size_t)kk * p.n_heads];
    float a0[4] = {0.f, 0.f, 0.f, 0.f}, a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < LIP_XBLOCK; kk += 2) {
        const float wa0 = __uint_as_float(wv[kk] << 16), wa1 = __uint_as_float(wv[kk] & 0xffff0000u);
        const float wb0 = __uint_as_float(wv[kk + 1] << 16), wb1 = __uint_as_float(wv[kk + 1] & 0xffff0000u);
        const float pa = bf16_bits_to_f32(pv[kk]);
        const float pb = bf16_bits_to_f32(pv[kk + 1]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t xv = xr[t][kk >> 1];
            const float xa = __uint_as_float(xv << 16), xb = __uint_as_float(xv & 0xffff0000u);
            a0[t] = __builtin_fmaf(xa, wa0, a0[t]);
            a1[t] = __builtin_fmaf(xa, wa1, a1[t]);
            a2[t] = __builtin_fmaf(xa, pa, a2[t]);
            a0[t] = __builtin_fmaf(xb, wb0, a0[t]);
            a1[t] = __builtin_fmaf(xb, wb1, a1[t]);
            a2[t] = __builtin_fmaf(xb, pb, a2[t]);
        }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t0 + t < p.T) {
            float *dst = p.xpart + ((size_t)c * p.T + t0 + t) * LIP_XCOLS;
            f32x2 v = {a0[t], a1[t]};
            *reinterpret_cast<f32x2 *>(dst + 2 * l) = v;
            if (pl) dst[LIP_DIM + l] = a2[t];
        }
    }
}

template <int STEPS>
__global__ __launch_bounds__(64) void lip_linear_kernel(const LipParams p, const int q_jobs)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lip_smem[];
    const int job = blockIdx.x;
    if (job < q_jobs) q_linear_job<STEPS>(p, lip_smem, job);
    else x_linear_job(p, job - q_jobs);
}

// ---------------------------------------------------------------------------------------------
// Second launch.

__device__ __forceinline__ float wave_max_f32(float v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}

// sum of the wave's 128 values (two per lane, neighbours) as a balanced tree over neighbours
__device__ __forceinline__ float pair_tree_sum(const float v0, const float v1)
{
    float s = __fadd_rn(v0, v1);
#pragma unroll
    for (int m = 1; m <= 32; m <<= 1) s = __fadd_rn(s, __shfl_xor(s, m));
    return s;
}

// rope on channels 0..63 (lanes 0..31 hold channels 2l, 2l+1); the rotation partner of channel i is
// i+32 (negated) for i < 32 and i-32 otherwise: lane l ^ 16.  Results rounded to bf16.
__device__ __forceinline__ void rope_pair(float &v0, float &v1, const uint16_t *cos, const uint16_t *sin, const int t, const int l)
{
    const float p0 = __shfl_xor(v0, 16);
    const float p1 = __shfl_xor(v1, 16);
    if (l < 32) {
        const uint32_t c = reinterpret_cast<const uint32_t *>(cos + (size_t)t * LIP_ROPE)[l];
        const uint32_t s = reinterpret_cast<const uint32_t *>(sin + (size_t)t * LIP_ROPE)[l];
        const float sg = l < 16 ? -1.0f : 1.0f;
        // both products are exact, so the fused form rounds once, like product + product
        const float r0 = __builtin_fmaf(v0, __uint_as_float(c << 16), (sg * p0) * __uint_as_float(s << 16));
        const float r1 = __builtin_fmaf(v1, __uint_as_float(c & 0xffff0000u), (sg * p1) * __uint_as_float(s & 0xffff0000u));
        v0 = bf16_round_f32(r0);
        v1 = bf16_round_f32(r1);
    }
}

// y[j] = sum_i a[i] * H[i][j], i ascending; lane l computes columns 2l and 2l+1.  a: this wave's 128
// floats in LDS, hmat: the matrix in LDS as stored (row-major bf16).
__device__ __forceinline__ void hadamard_pair(const float *a, const uint32_t *hmat, const int l, float &y0, float &y1)
{
    float o0 = 0.f, o1 = 0.f;
#pragma unroll 4
    for (int i = 0; i < LIP_DIM; i += 4) {
        const f32x4 av = *reinterpret_cast<const f32x4 *>(a + i);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t hv = hmat[(i + u) * 64 + l];
            o0 = __builtin_fmaf(av[u], __uint_as_float(hv << 16), o0);
            o1 = __builtin_fmaf(av[u], __uint_as_float(hv & 0xffff0000u), o1);
        }
    }
    y0 = bf16_round_f32(o0);
    y1 = bf16_round_f32(o1);
}

// symmetric int8 quantisation of the wave's 128 values; returns the packed byte pair and the scale
__device__ __forceinline__ uint16_t quant_pair(const float y0, const float y1, uint16_t &scale_f16)
{
    const float amax = wave_max_f32(fmaxf(fabsf(y0), fabsf(y1)));
    if (amax > 0.f) {
        const float s = __fdiv_rn(127.0f, amax);
        const int q0 = (int)rintf(__fmul_rn(y0, s));
        const int q1 = (int)rintf(__fmul_rn(y1, s));
        scale_f16 = (uint16_t)(pack_f16x2(__fdiv_rn(1.0f, s), 0.f) & 0xffffu);
        return (uint16_t)((q0 & 0xff) | ((q1 & 0xff) << 8));
    }
    scale_f16 = 0;
    return 0;
}

constexpr int FIN_WAVES = 16;

__device__ __forceinline__ void stage_matrix(uint32_t *dst, const uint16_t *src)
{
    const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
    u32x4 *d = reinterpret_cast<u32x4 *>(dst);
#pragma unroll
    for (int i = 0; i < 2; ++i) d[i * 1024 + threadIdx.x] = s[i * 1024 + threadIdx.x];
}

// Workgroups [0, q_wgs): sixteen query rows (token, head) each, one per wave.
// Workgroups [q_wgs, q_wgs + T): one token each -- waves add the groups of block sums over the hidden
// axis (one group of eight blocks per wave and round), then wave 0 finishes the key row and wave 1 the
// weights row.
__global__ __launch_bounds__(64 * FIN_WAVES) void lip_finish_kernel(const LipParams p, const int q_wgs)
{
    __shared__ __attribute__((aligned(16))) uint32_t hmat[LIP_DIM * 64];
    __shared__ __attribute__((aligned(16))) float arow[FIN_WAVES][LIP_DIM];
    __shared__ __attribute__((aligned(16))) float gsum[LIP_MAX_XGROUPS][LIP_XCOLS];
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ncols = p.n_heads * LIP_DIM;
    const int wg = blockIdx.x;

    if (wg < q_wgs) {
        stage_matrix(hmat, p.hq);
        const int row = wg * FIN_WAVES + w;            // (token, head)
        const bool live = row < p.T * p.n_heads;
        const int t = live ? row / p.n_heads : 0;
        const int head = live ? row % p.n_heads : 0;
        const int col = head * LIP_DIM + 2 * l;
        int s0 = 0, s1 = 0;
#pragma unroll
        for (int kq = 0; kq < LIP_KSPLIT; ++kq) {
            const int2 v = *reinterpret_cast<const int2 *>(p.qpart + ((size_t)kq * p.T + t) * ncols + col);
            s0 += v.x;
            s1 += v.y;
        }
        const float ts = p.q_norm_scale[t];
        const f32x2 cs = *reinterpret_cast<const f32x2 *>(p.w_qb_scale + col);
        float v0 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s0, ts), cs[0]));
        float v1 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s1, ts), cs[1]));
        rope_pair(v0, v1, p.cos, p.sin, t, l);
        f32x2 av = {v0, v1};
        *reinterpret_cast<f32x2 *>(&arow[w][2 * l]) = av;
        __syncthreads();
        float y0, y1;
        hadamard_pair(arow[w], hmat, l, y0, y1);
        uint16_t sc;
        const uint16_t q = quant_pair(y0, y1, sc);
        if (live) {
            reinterpret_cast<uint16_t *>(p.q_int8 + (size_t)row * LIP_DIM)[l] = q;
            if (l == 0) p.q_scale[row] = sc;
        }
        return;
    }

    const int t = wg - q_wgs;
    const int nblk = p.h / LIP_XBLOCK;
    const int ngroups = (nblk + LIP_XGROUP - 1) / LIP_XGROUP;
    stage_matrix(hmat, p.hk);
    const bool pl = l < p.n_heads;
    for (int g = w; g < ngroups; g += FIN_WAVES) {
        const float *src = p.xpart + ((size_t)g * LIP_XGROUP * p.T + t) * LIP_XCOLS;
        const int nb = nblk - g * LIP_XGROUP < LIP_XGROUP ? nblk - g * LIP_XGROUP : LIP_XGROUP;
        f32x2 kv[LIP_XGROUP];
        float wv[LIP_XGROUP];
#pragma unroll
        for (int i = 0; i < LIP_XGROUP; ++i) {
            const float *r = src + (size_t)(i < nb ? i : 0) * p.T * LIP_XCOLS;
            kv[i] = *reinterpret_cast<const f32x2 *>(r + 2 * l);
            wv[i] = r[LIP_DIM + (pl ? l : 0)];
        }
        float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int i = 0; i < LIP_XGROUP; ++i) {
            if (i < nb) {
                s0 = __fadd_rn(s0, kv[i][0]);
                s1 = __fadd_rn(s1, kv[i][1]);
                s2 = __fadd_rn(s2, wv[i]);
            }
        }
        f32x2 sv = {s0, s1};
        *reinterpret_cast<f32x2 *>(&gsum[g][2 * l]) = sv;
        gsum[g][LIP_DIM + l] = s2;
    }
    __syncthreads();
    if (w == 0) {
        float v0 = 0.f, v1 = 0.f;
        for (int g = 0; g < ngroups; ++g) {
            const f32x2 v = *reinterpret_cast<const f32x2 *>(&gsum[g][2 * l]);
            v0 = __fadd_rn(v0, v[0]);
            v1 = __fadd_rn(v1, v[1]);
        }
        // layer norm over the 128 channels
        const float mean = __fmul_rn(pair_tree_sum(v0, v1), 1.0f / LIP_DIM);
        const float d0 = __fsub_rn(v0, mean), d1 = __fsub_rn(v1, mean);
        const float var = __fmul_rn(pair_tree_sum(__fmul_rn(d0, d0), __fmul_rn(d1, d1)), 1.0f / LIP_DIM);
        const float sd = __fsqrt_rn(__fadd_rn(var, p.eps));
        const uint32_t g = reinterpret_cast<const uint32_t *>(p.gamma)[l];
        const uint32_t b = reinterpret_cast<const uint32_t *>(p.beta)[l];
        v0 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d0, sd), __uint_as_float(g << 16)), __uint_as_float(b << 16)));
        v1 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d1, sd), __uint_as_float(g & 0xffff0000u)), __uint_as_float(b & 0xffff0000u)));
        rope_pair(v0, v1, p.cos, p.sin, t, l);
        f32x2 av = {v0, v1};
        *reinterpret_cast<f32x2 *>(&arow[0][2 * l]) = av;
        float y0, y1;
        hadamard_pair(arow[0], hmat, l, y0, y1);       // same wave wrote arow[0]: LDS operations of a wave stay in order
        uint16_t sc;
        const uint16_t q = quant_pair(y0, y1, sc);
        const long long dst = p.k_cache_index[t];
        if (dst >= 0 && dst < p.cache_rows) {
            reinterpret_cast<uint16_t *>(p.k_cache + (size_t)dst * LIP_DIM)[l] = q;
            if (l == 0) p.k_cache_scale[dst] = sc;
        }
    } else if (w == 1 && pl) {
        float v = 0.f;
        for (int g = 0; g < ngroups; ++g) v = __fadd_rn(v, gsum[g][LIP_DIM + l]);
        v = __fmul_rn(__fmul_rn(bf16_round_f32(v), p.w_mul0), p.w_mul1);
        p.weights[(size_t)t * p.n_heads + l] = (uint16_t)(pack_f16x2(v, 0.f) & 0xffffu);
    }
}

}  // namespace

hipError_t lip_launch(const LipParams &p, hipStream_t stream)
{
    const int steps = p.q_lora / LIP_KSPLIT / 32;
    const int tblocks = (p.T + 31) / 32;
    const int q_jobs = p.n_heads * LIP_KSPLIT * tblocks;
    const int x_jobs = (p.h / LIP_XBLOCK) * ((p.T + 3) / 4);
    const dim3 grid1((unsigned)(q_jobs + x_jobs)), block1(64);
    const size_t lds = (size_t)steps * 32 * 128 + (size_t)steps * 1024;
    switch (steps) {
    case 4: hipLaunchKernelGGL(lip_linear_kernel<4>, grid1, block1, lds, stream, p, q_jobs); break;
    case 8: hipLaunchKernelGGL(lip_linear_kernel<8>, grid1, block1, lds, stream, p, q_jobs); break;
    case 12: hipLaunchKernelGGL(lip_linear_kernel<12>, grid1, block1, lds, stream, p, q_jobs); break;
    default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int q_wgs = (p.T * p.n_heads + FIN_WAVES - 1) / FIN_WAVES;
    hipLaunchKernelGGL(lip_finish_kernel, dim3((unsigned)(q_wgs + p.T)), dim3(64 * FIN_WAVES), 0, stream, p, q_wgs);
    return hipGetLastError();
}

}  // namespace pto
