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
//   lip_linear_kernel   workgroups of four independent waves.  Two of them share a query job (head,
//                       quarter of the reduction axis, block of 32 tokens), one half each: the tile of
//                       w_qb (rows x 128 bytes) and the token rows travel to LDS by LDS-DMA, all
//                       requests issued up front; 32-row steps are consumed as their requests land
//                       (they complete in order): 4x4 byte transposes (v_perm_b32) turn the row-major
//                       tile into v_mfma_i32_32x32x32_i8 operands.  The two halves are added through
//                       LDS and the partial int32 sums go to the workspace.  The other two waves take
//                       hidden-axis jobs (block of 64 rows of wk or of w_proj, 4 tokens): fp32 FMAs
//                       with the hidden states as scalar operands; block sums go to the workspace.
//   lip_finish_kernel   Query rows, one per wave: add the four partial sums, de-quantise, rope,
//                       Hadamard (matrix staged in LDS once per workgroup), quantise, store.  Tokens,
//                       one workgroup each: waves add the groups of block sums, then one wave finishes
//                       the key row (layer norm, rope, Hadamard, quantise, scatter) and one the weights.
#include "lip_kernels.h"
#include "prolog_common.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

static_assert(LIP_KSPLIT == QPROJ_KSPLIT, "workspace sizing and the projection job disagree");

// ---------------------------------------------------------------------------------------------
// Hidden-axis jobs: block c of 64 rows, tokens t0, t0+1.  Even jobs take wk (lane l: columns 2l,
// 2l+1), odd jobs w_proj (lane l: column l).  The block of weights (contiguous in memory) travels to
// the wave's LDS region by LDS-DMA, the two token slices are converted to fp32 on the way in; the
// product loop reads weights per lane and the hidden states as broadcasts.
constexpr int XW_BYTES = LIP_XBLOCK * LIP_DIM * 2;     // 16 KiB: a block of wk
constexpr int XTOK = 2;                               // tokens per hidden-axis job
constexpr int X_REGION_BYTES = XW_BYTES + XTOK * LIP_XBLOCK * 4;
constexpr int LIN_XWAVES = 4;

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
    {   // lane l: hidden states k0 + 2*(l%32), +1 of token t0 + l/32
        const int t = t0 + (l >> 5);
        const int tt = t < p.T ? t : p.T - 1;
        const uint32_t xv = reinterpret_cast<const uint32_t *>(p.x + (size_t)tt * p.h + k0)[l & 31];
        f32x2 v = {__uint_as_float(xv << 16), __uint_as_float(xv & 0xffff0000u)};
        *reinterpret_cast<f32x2 *>(xs + (l >> 5) * LIP_XBLOCK + 2 * (l & 31)) = v;
    }
    VM_WAIT(0);
    // the wave reads back only what it wrote or requested itself: no barrier

    if (!proj) {
        const uint32_t *wl = reinterpret_cast<const uint32_t *>(region) + l;
        float a0[XTOK] = {0.f, 0.f}, a1[XTOK] = {0.f, 0.f};
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
        float a2[XTOK] = {0.f, 0.f};
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

template <int HS>
constexpr int lin_lds_bytes()
{
    return 2 * lin_region_bytes<HS>() + LIN_XWAVES * X_REGION_BYTES;
}

// Workgroup of six waves, no dependencies among them except the final pairwise sum of the two query
// waves: waves 0 and 1 run the two halves of query job blockIdx.x, waves 2..5 walk the hidden-axis jobs.
template <int HS>
__global__ __launch_bounds__(128 + 64 * LIN_XWAVES) void lip_linear_kernel(const LipParams p, const int q_jobs, const int x_jobs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lip_smem[lin_lds_bytes<HS>()];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = threadIdx.x & 63;
    const int job = blockIdx.x;
    const bool qwave = w < 2 && job < q_jobs;
    uint8_t *region = lip_smem + (w & 1) * lin_region_bytes<HS>();
    i32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;

    const QProj qp = {p.q_norm, p.w_qb, p.qpart, p.T, p.q_lora, p.n_heads};
    if (qwave) {
        q_half_job<HS>(qp, region, job, w, acc);
        if (w == 1) q_pair_park(region, l, acc);
    } else if (w >= 2) {
        uint8_t *xregion = lip_smem + 2 * lin_region_bytes<HS>() + (w - 2) * X_REGION_BYTES;
        for (int j = job * LIN_XWAVES + (w - 2); j < x_jobs; j += gridDim.x * LIN_XWAVES) x_linear_job(p, xregion, j);
    }
    __syncthreads();
    if (qwave && w == 0) q_pair_store<HS>(qp, lip_smem, job, l, acc);
}

// ---------------------------------------------------------------------------------------------
// Second launch.

// rope on channels 0..63 (lanes 0..31 hold channels 2l, 2l+1); the rotation partner of channel i is
// i+32 (negated) for i < 32 and i-32 otherwise: lane l ^ 16.  Results rounded to bf16.
__device__ __forceinline__ void rope_pair(float &v0, float &v1, const uint32_t c, const uint32_t s, const int l)
{
    const float p0 = xor16_f32(v0, l);
    const float p1 = xor16_f32(v1, l);
    if (l < 32) {
        const float sg = l < 16 ? -1.0f : 1.0f;
        // both products are exact, so the fused form rounds once, like product + product
        const float r0 = __builtin_fmaf(v0, __uint_as_float(c << 16), (sg * p0) * __uint_as_float(s << 16));
        const float r1 = __builtin_fmaf(v1, __uint_as_float(c & 0xffff0000u), (sg * p1) * __uint_as_float(s & 0xffff0000u));
        v0 = bf16_round_f32(r0);
        v1 = bf16_round_f32(r1);
    }
}
// the cos / sin pair of lane l (channels 2l, 2l+1 of token t); lanes 32..63 read lane l-32's, unused
__device__ __forceinline__ uint32_t rope_coef(const uint16_t *tab, const int t, const int l)
{
    return reinterpret_cast<const uint32_t *>(tab + (size_t)t * LIP_ROPE)[l & 31];
}

// y[j] = sum_i a[i] * H[i][j], i ascending; lane l computes columns 2l and 2l+1.  a: this wave's 128
// floats in LDS, hmat: the matrix in LDS as fp32, row-major.  Chunks of 16 rows are read one chunk
// ahead of the multiply-adds that consume them.
struct HadChunk {
    f32x4 a[4];
    f32x2 h[16];
};
__device__ __forceinline__ void had_load(HadChunk &c, const float *a, const float *hmat, const int l, const int i0)
{
#pragma unroll
    for (int u = 0; u < 4; ++u) c.a[u] = *reinterpret_cast<const f32x4 *>(a + i0 + 4 * u);
#pragma unroll
    for (int u = 0; u < 16; ++u) c.h[u] = *reinterpret_cast<const f32x2 *>(hmat + (i0 + u) * LIP_DIM + 2 * l);
}
__device__ __forceinline__ void had_fma(const HadChunk &c, float &o0, float &o1)
{
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        o0 = __builtin_fmaf(c.a[u >> 2][u & 3], c.h[u][0], o0);
        o1 = __builtin_fmaf(c.a[u >> 2][u & 3], c.h[u][1], o1);
    }
}
__device__ __forceinline__ void hadamard_pair(const float *a, const float *hmat, const int l, float &y0, float &y1)
{
    float o0 = 0.f, o1 = 0.f;
    HadChunk c0, c1;
    had_load(c0, a, hmat, l, 0);
#pragma unroll 1
    for (int i = 0; i < LIP_DIM; i += 32) {
        had_load(c1, a, hmat, l, i + 16);
        had_fma(c0, o0, o1);
        had_load(c0, a, hmat, l, i + 32 < LIP_DIM ? i + 32 : 0);
        had_fma(c1, o0, o1);
    }
    y0 = bf16_round_f32(o0);
    y1 = bf16_round_f32(o1);
}

// symmetric int8 quantisation of the wave's 128 values; returns the packed byte pair and the fp16 scale
__device__ __forceinline__ uint16_t quant_pair(const float y0, const float y1, uint16_t &scale_f16)
{
    const float amax = wave_max_f32(fmaxf(fabsf(y0), fabsf(y1)));
    float deq;
    const uint16_t q = quant_pair_amax(y0, y1, amax, deq);
    scale_f16 = (uint16_t)(pack_f16x2(deq, 0.f) & 0xffffu);
    return q;
}

constexpr int FIN_WAVES = 8;

// the 128x128 bf16 matrix, widened to fp32, into LDS
__device__ __forceinline__ void stage_matrix(float *dst, const uint16_t *src)
{
    const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
    constexpr int NT = 64 * FIN_WAVES;
#pragma unroll
    for (int i = 0; i < 2048 / NT; ++i) {
        const u32x4 v = s[i * NT + threadIdx.x];
        f32x4 lo = {__uint_as_float(v[0] << 16), __uint_as_float(v[0] & 0xffff0000u), __uint_as_float(v[1] << 16),
                    __uint_as_float(v[1] & 0xffff0000u)};
        f32x4 hi = {__uint_as_float(v[2] << 16), __uint_as_float(v[2] & 0xffff0000u), __uint_as_float(v[3] << 16),
                    __uint_as_float(v[3] & 0xffff0000u)};
        f32x4 *d = reinterpret_cast<f32x4 *>(dst + (size_t)(i * NT + threadIdx.x) * 8);
        d[0] = lo;
        d[1] = hi;
    }
}

// Workgroups [0, q_wgs): FIN_WAVES query rows (token, head) each, one per wave.
// Workgroups [q_wgs, q_wgs + T): one token each -- waves add the groups of block sums over the hidden
// axis (two groups of eight blocks per wave and round), then wave 0 finishes the key row and wave 1 the
// weights row.
__global__ __launch_bounds__(64 * FIN_WAVES) void lip_finish_kernel(const LipParams p, const int q_wgs)
{
    __shared__ __attribute__((aligned(16))) float hmat[LIP_DIM * LIP_DIM];
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
        const uint32_t rc = rope_coef(p.cos, t, l), rs = rope_coef(p.sin, t, l);
        float v0 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s0, ts), cs[0]));
        float v1 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s1, ts), cs[1]));
        rope_pair(v0, v1, rc, rs, l);
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
    // everything wave 0 needs later is requested now
    const uint32_t rc = rope_coef(p.cos, t, l), rs = rope_coef(p.sin, t, l);
    const uint32_t gm = reinterpret_cast<const uint32_t *>(p.gamma)[l];
    const uint32_t bt = reinterpret_cast<const uint32_t *>(p.beta)[l];
    const long long dst = p.k_cache_index[t];
    for (int g0 = w; g0 < ngroups; g0 += 2 * FIN_WAVES) {
        f32x2 kv[2][LIP_XGROUP];
        float wv[2][LIP_XGROUP];
        int nb[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int g = g0 + u * FIN_WAVES;
            const int left = nblk - g * LIP_XGROUP;
            nb[u] = left < 0 ? 0 : (left < LIP_XGROUP ? left : LIP_XGROUP);
            const float *src = p.xpart + ((size_t)(nb[u] ? g : 0) * LIP_XGROUP * p.T + t) * LIP_XCOLS;
#pragma unroll
            for (int i = 0; i < LIP_XGROUP; ++i) {
                const float *r = src + (size_t)(i < nb[u] ? i : 0) * p.T * LIP_XCOLS;
                kv[u][i] = *reinterpret_cast<const f32x2 *>(r + 2 * l);
                wv[u][i] = r[LIP_DIM + (pl ? l : 0)];
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (nb[u] == 0) continue;
            float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int i = 0; i < LIP_XGROUP; ++i) {
                if (i < nb[u]) {
                    s0 = __fadd_rn(s0, kv[u][i][0]);
                    s1 = __fadd_rn(s1, kv[u][i][1]);
                    s2 = __fadd_rn(s2, wv[u][i]);
                }
            }
            const int g = g0 + u * FIN_WAVES;
            f32x2 sv = {s0, s1};
            *reinterpret_cast<f32x2 *>(&gsum[g][2 * l]) = sv;
            gsum[g][LIP_DIM + l] = s2;
        }
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
        const float sd = __builtin_sqrtf(__fadd_rn(var, p.eps));   // correctly rounded (__fsqrt_rn is the 1-ulp hardware root here)
        v0 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d0, sd), __uint_as_float(gm << 16)), __uint_as_float(bt << 16)));
        v1 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d1, sd), __uint_as_float(gm & 0xffff0000u)), __uint_as_float(bt & 0xffff0000u)));
        rope_pair(v0, v1, rc, rs, l);
        f32x2 av = {v0, v1};
        *reinterpret_cast<f32x2 *>(&arow[0][2 * l]) = av;
        float y0, y1;
        hadamard_pair(arow[0], hmat, l, y0, y1);       // same wave wrote arow[0]: LDS operations of a wave stay in order
        uint16_t sc;
        const uint16_t q = quant_pair(y0, y1, sc);
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
    const int x_jobs = 2 * (p.h / LIP_XBLOCK) * ((p.T + XTOK - 1) / XTOK);
    // enough workgroups that each hidden-axis wave gets about one job, never fewer than the query jobs
    int wgs = (x_jobs + LIN_XWAVES - 1) / LIN_XWAVES;
    wgs = wgs > 4096 ? 4096 : wgs;
    wgs = wgs > q_jobs ? wgs : q_jobs;
    const dim3 grid1((unsigned)wgs), block1(128 + 64 * LIN_XWAVES);
    switch (steps) {
    case 4: hipLaunchKernelGGL(lip_linear_kernel<2>, grid1, block1, 0, stream, p, q_jobs, x_jobs); break;
    case 8: hipLaunchKernelGGL(lip_linear_kernel<4>, grid1, block1, 0, stream, p, q_jobs, x_jobs); break;
    case 12: hipLaunchKernelGGL(lip_linear_kernel<6>, grid1, block1, 0, stream, p, q_jobs, x_jobs); break;
    default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int q_wgs = (p.T * p.n_heads + FIN_WAVES - 1) / FIN_WAVES;
    hipLaunchKernelGGL(lip_finish_kernel, dim3((unsigned)(q_wgs + p.T)), dim3(64 * FIN_WAVES), 0, stream, p, q_wgs);
    return hipGetLastError();
}

}  // namespace pto
