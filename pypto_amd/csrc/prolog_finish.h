// The last launch of each of the two prologs (query rows finished: rope, Hadamard / absorb product,
// quantisation; key row and head weights of the indexer) as device functions over an LDS pool, so that
// the same code runs as a launch of its own and, for the fused operator, side by side in one launch.
// Included by lip_kernels.hip, mlap_kernels.hip and prolog_fused.hip after prolog_common.h.
#pragma once
#include "lip_kernels.h"
#include "mlap_kernels.h"
#include "prolog_common.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

// the de-quantised int8 projection for columns col, col + 1 of token t, as bf16-valued floats: the unsplit form left
// them that way; the split form's partial sums are added and de-quantised here
__device__ __forceinline__ void q_value2(const int32_t *part, const int splits, const int T, const int t, const int ncols, const int col,
                                         const float ts, const float cs0, const float cs1, float &v0, float &v1)
{
    if (splits == 1) {
        const uint32_t v = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint16_t *>(part) + (size_t)t * ncols + col);
        v0 = __uint_as_float(v << 16);
        v1 = __uint_as_float(v & 0xffff0000u);
        return;
    }
    int s0 = 0, s1 = 0;
#pragma unroll
    for (int kq = 0; kq < QPROJ_KSPLIT; ++kq) {
        const int2 v = *reinterpret_cast<const int2 *>(part + ((size_t)kq * T + t) * ncols + col);
        s0 += v.x;
        s1 += v.y;
    }
    v0 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s0, ts), cs0));
    v1 = bf16_round_f32(__fmul_rn(__fmul_rn((float)s1, ts), cs1));
}

// ------------------------------------------------------------------------------ indexer prolog
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
// floats in LDS, hmat: the matrix in LDS as it is in memory (bf16, row-major; widened on the way into the
// registers, which costs two instructions per row and halves the workgroup's LDS).  Chunks of 16 rows are read
// one chunk ahead of the multiply-adds that consume them.
struct HadChunk {
    f32x4 a[4];
    f32x2 h[16];
};
__device__ __forceinline__ void had_load(HadChunk &c, const float *a, const uint16_t *hmat, const int l, const int i0)
{
#pragma unroll
    for (int u = 0; u < 4; ++u) c.a[u] = *reinterpret_cast<const f32x4 *>(a + i0 + 4 * u);
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const uint32_t x = *reinterpret_cast<const uint32_t *>(hmat + (i0 + u) * LIP_DIM + 2 * l);
        c.h[u][0] = __uint_as_float(x << 16);
        c.h[u][1] = __uint_as_float(x & 0xffff0000u);
    }
}
__device__ __forceinline__ void had_fma(const HadChunk &c, float &o0, float &o1)
{
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        o0 = __builtin_fmaf(c.a[u >> 2][u & 3], c.h[u][0], o0);
        o1 = __builtin_fmaf(c.a[u >> 2][u & 3], c.h[u][1], o1);
    }
}
__device__ __forceinline__ void hadamard_pair(const float *a, const uint16_t *hmat, const int l, float &y0, float &y1)
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

// the 128x128 bf16 matrix into LDS, as it is (2048 pieces of 16 bytes over the workgroup's FIN_WAVES waves)
__device__ __forceinline__ void stage_matrix(uint16_t *dst, const uint16_t *src)
{
    const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
    u32x4 *d = reinterpret_cast<u32x4 *>(dst);
    constexpr int NT = 64 * FIN_WAVES;
#pragma unroll
    for (int i = 0; i < 2048 / NT; ++i) d[i * NT + threadIdx.x] = s[i * NT + threadIdx.x];
}

// a key row from its sums over the hidden axis (lane l: channels 2l, 2l+1): layer norm, rope, Hadamard product with the
// matrix in LDS (a: this wave's 128 floats of LDS), quantisation, scatter to cache row dst (skipped if out of range)
__device__ __forceinline__ void lip_key_row(const LipParams &p, const uint16_t *hmat, float *a, float v0, float v1, const uint32_t rc,
                                            const uint32_t rs, const uint32_t gm, const uint32_t bt, const long long dst, const int l)
{
    const float mean = __fmul_rn(pair_tree_sum(v0, v1), 1.0f / LIP_DIM);
    const float d0 = __fsub_rn(v0, mean), d1 = __fsub_rn(v1, mean);
    const float var = __fmul_rn(pair_tree_sum(__fmul_rn(d0, d0), __fmul_rn(d1, d1)), 1.0f / LIP_DIM);
    const float sd = __builtin_sqrtf(__fadd_rn(var, p.eps));   // correctly rounded (__fsqrt_rn is the 1-ulp hardware root here)
    v0 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d0, sd), __uint_as_float(gm << 16)), __uint_as_float(bt << 16)));
    v1 = bf16_round_f32(__fadd_rn(__fmul_rn(__fdiv_rn(d1, sd), __uint_as_float(gm & 0xffff0000u)), __uint_as_float(bt & 0xffff0000u)));
    rope_pair(v0, v1, rc, rs, l);
    f32x2 av = {v0, v1};
    *reinterpret_cast<f32x2 *>(&a[2 * l]) = av;
    float y0, y1;
    hadamard_pair(a, hmat, l, y0, y1);                 // the same wave wrote a: LDS operations of a wave stay in order
    uint16_t sc;
    const uint16_t q = quant_pair(y0, y1, sc);
    if (dst >= 0 && dst < p.cache_rows) {
        reinterpret_cast<uint16_t *>(p.k_cache + (size_t)dst * LIP_DIM)[l] = q;
        if (l == 0) p.k_cache_scale[dst] = sc;
    }
}
// head weight l of token t from its sum over the hidden axis
__device__ __forceinline__ void lip_weight(const LipParams &p, const int t, const int l, float v)
{
    v = __fmul_rn(__fmul_rn(bf16_round_f32(v), p.w_mul0), p.w_mul1);
    p.weights[(size_t)t * p.n_heads + l] = (uint16_t)(pack_f16x2(v, 0.f) & 0xffffu);
}

// Workgroups [0, q_wgs): FIN_WAVES query rows (token, head) each, one per wave.
// Workgroups [q_wgs, q_wgs + T): one token each -- waves add the groups of block sums over the hidden
// axis (two groups of eight blocks per wave and round), then wave 0 finishes the key row and wave 1 the
// weights row.
constexpr int LIP_FIN_LDS = LIP_DIM * LIP_DIM * 2 + FIN_WAVES * LIP_DIM * 4 + LIP_MAX_XGROUPS * LIP_XCOLS * 4;   // 55 296 bytes

// The work of workgroup wg of the second launch (64 * FIN_WAVES threads), in LIP_FIN_LDS bytes of LDS at lds.
__device__ __forceinline__ void lip_finish_body(const LipParams &p, const int q_wgs, const int wg, uint8_t *lds)
{
    uint16_t *hmat = reinterpret_cast<uint16_t *>(lds);
    float(*arow)[LIP_DIM] = reinterpret_cast<float(*)[LIP_DIM]>(lds + LIP_DIM * LIP_DIM * 2);
    float(*gsum)[LIP_XCOLS] = reinterpret_cast<float(*)[LIP_XCOLS]>(lds + LIP_DIM * LIP_DIM * 2 + FIN_WAVES * LIP_DIM * 4);
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ncols = p.n_heads * LIP_DIM;

    if (wg < q_wgs) {
        stage_matrix(hmat, p.hq);
        const int row = wg * FIN_WAVES + w;            // (token, head)
        const bool live = row < p.T * p.n_heads;
        const int t = live ? row / p.n_heads : 0;
        const int head = live ? row % p.n_heads : 0;
        const int col = head * LIP_DIM + 2 * l;
        const float ts = p.q_norm_scale[t];
        const f32x2 cs = *reinterpret_cast<const f32x2 *>(p.w_qb_scale + col);
        const uint32_t rc = rope_coef(p.cos, t, l), rs = rope_coef(p.sin, t, l);
        float v0, v1;
        q_value2(p.qpart, qproj_splits(p.T), p.T, t, ncols, col, ts, cs[0], cs[1], v0, v1);
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
    const bool group_rows = lip_x_group_rows(p);       // the rows are group sums already
    const int nblk = group_rows ? 0 : lip_xrows(p);
    const int ngroups = group_rows ? lip_xrows(p) : (nblk + LIP_XGROUP - 1) / LIP_XGROUP;
    stage_matrix(hmat, p.hk);
    const bool pl = l < p.n_heads;
    // everything wave 0 needs later is requested now
    const uint32_t rc = rope_coef(p.cos, t, l), rs = rope_coef(p.sin, t, l);
    const uint32_t gm = reinterpret_cast<const uint32_t *>(p.gamma)[l];
    const uint32_t bt = reinterpret_cast<const uint32_t *>(p.beta)[l];
    const long long dst = p.k_cache_index[t];
    if (group_rows) {
        for (int g = w; g < ngroups; g += FIN_WAVES) {
            const float *r = p.xpart + ((size_t)g * p.T + t) * LIP_XCOLS;
            *reinterpret_cast<f32x2 *>(&gsum[g][2 * l]) = *reinterpret_cast<const f32x2 *>(r + 2 * l);
            gsum[g][LIP_DIM + l] = r[LIP_DIM + (pl ? l : 0)];
        }
    }
    for (int g0 = w; g0 < ngroups && !group_rows; g0 += 2 * FIN_WAVES) {
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
        lip_key_row(p, hmat, arow[0], v0, v1, rc, rs, gm, bt, dst, l);
    } else if (w == 1 && pl) {
        float v = 0.f;
        for (int g = 0; g < ngroups; ++g) v = __fadd_rn(v, gsum[g][LIP_DIM + l]);
        lip_weight(p, t, l, v);
    }
}

// The key rows and weights at prefill sizes: a workgroup of FIN_WAVES waves takes FIN_WAVES tokens, one per wave (the
// matrix is staged once for all of them instead of once per token, and the rows are finished side by side instead of
// by one wave per workgroup).  A wave adds its token's partial rows in registers, in the order of the form they come
// in: group sums ascending, or blocks / ranges ascending into groups of eight and the groups ascending.
constexpr int LIP_FINT_LDS = LIP_DIM * LIP_DIM * 2 + FIN_WAVES * LIP_DIM * 4;

__device__ __forceinline__ void lip_finish_tokens_prefill_body(const LipParams &p, const int wg, uint8_t *lds)
{
    uint16_t *hmat = reinterpret_cast<uint16_t *>(lds);
    float(*arow)[LIP_DIM] = reinterpret_cast<float(*)[LIP_DIM]>(lds + LIP_DIM * LIP_DIM * 2);
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = wg * FIN_WAVES + w;
    const bool live = t < p.T;
    const int tt = live ? t : p.T - 1;
    stage_matrix(hmat, p.hk);
    const bool pl = l < p.n_heads;
    const uint32_t rc = rope_coef(p.cos, tt, l), rs = rope_coef(p.sin, tt, l);
    const uint32_t gm = reinterpret_cast<const uint32_t *>(p.gamma)[l];
    const uint32_t bt = reinterpret_cast<const uint32_t *>(p.beta)[l];
    const long long dst = live ? p.k_cache_index[tt] : -1;
    const bool group_rows = lip_x_group_rows(p);
    const int nrows = lip_xrows(p);
    const float *src = p.xpart + (size_t)tt * LIP_XCOLS;
    const size_t rstride = (size_t)p.T * LIP_XCOLS;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f;
    for (int g0 = 0; g0 < nrows; g0 += LIP_XGROUP) {
        f32x2 kv[LIP_XGROUP];
        float wv[LIP_XGROUP];
        const int nb = nrows - g0 < LIP_XGROUP ? nrows - g0 : LIP_XGROUP;
#pragma unroll
        for (int i = 0; i < LIP_XGROUP; ++i) {
            const float *r = src + (size_t)(g0 + (i < nb ? i : 0)) * rstride;
            kv[i] = *reinterpret_cast<const f32x2 *>(r + 2 * l);
            wv[i] = r[LIP_DIM + (pl ? l : 0)];
        }
        if (group_rows) {
#pragma unroll
            for (int i = 0; i < LIP_XGROUP; ++i) {
                if (i < nb) {
                    v0 = __fadd_rn(v0, kv[i][0]);
                    v1 = __fadd_rn(v1, kv[i][1]);
                    v2 = __fadd_rn(v2, wv[i]);
                }
            }
        } else {
            float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int i = 0; i < LIP_XGROUP; ++i) {
                if (i < nb) {
                    s0 = __fadd_rn(s0, kv[i][0]);
                    s1 = __fadd_rn(s1, kv[i][1]);
                    s2 = __fadd_rn(s2, wv[i]);
                }
            }
            v0 = __fadd_rn(v0, s0);
            v1 = __fadd_rn(v1, s1);
            v2 = __fadd_rn(v2, s2);
        }
    }
    __syncthreads();                                   // the matrix is staged
    lip_key_row(p, hmat, arow[w], v0, v1, rc, rs, gm, bt, dst, l);
    if (pl && live) lip_weight(p, t, l, v2);
}


// The query rows at prefill sizes with the Hadamard sums on the matrix cores: a workgroup of four waves stages the
// matrix once (rows padded to 272 bytes so that the four rows of a transposing read fall into different banks),
// then each wave walks passes of 32 rows (token, head): it de-quantises and rotates its rows, eight at a time, into
// its own bf16 operand buffer, takes O^T[j][row] = sum_i H^T[j][i] a^T[i][row] as 32 products
// (v_mfma_f32_32x32x16_bf16, A = the matrix read transposed, B = the rows), rounds to bf16, quantises each row
// (lanes l and l + 32 hold one row between them) and sends the int8 rows through its buffer so that they leave as
// whole 16-byte pieces.  All products are exact; the sums run in the cores' order instead of i ascending.
constexpr int QFP_WAVES = 4;
constexpr int QFP_HPITCH = 136;                        // elements between matrix rows in LDS
constexpr int QFP_APITCH = 136;                        // elements between operand rows
constexpr int QFP_OPITCH = 144;                        // bytes between int8 rows on their way out
constexpr int QFP_WAVE_BYTES = 32 * QFP_APITCH * 2;
constexpr int LIP_QFP_LDS = LIP_DIM * QFP_HPITCH * 2 + QFP_WAVES * QFP_WAVE_BYTES;   // 69 632 bytes
static_assert(32 * QFP_OPITCH <= QFP_WAVE_BYTES, "the int8 rows reuse the operand buffer");
static_assert(LIP_QFP_LDS <= 160 * 1024, "one workgroup fits a compute unit");

__device__ __forceinline__ void lip_finish_query_prefill_body(const LipParams &p, const int wg, const int nwg, uint8_t *lds)
{
    uint16_t *hmat = reinterpret_cast<uint16_t *>(lds);
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t *mine = lds + LIP_DIM * QFP_HPITCH * 2 + w * QFP_WAVE_BYTES;
    uint16_t *abf = reinterpret_cast<uint16_t *>(mine);
    {
        const u32x4 *s = reinterpret_cast<const u32x4 *>(p.hq);
        for (int i = threadIdx.x; i < LIP_DIM * LIP_DIM / 8; i += 64 * QFP_WAVES)
            *reinterpret_cast<u32x4 *>(hmat + (i >> 4) * QFP_HPITCH + (i & 15) * 8) = s[i];
    }
    __syncthreads();
    const int ncols = p.n_heads * LIP_DIM;
    const int nrows = p.T * p.n_heads;
    const int npass = (nrows + 31) / 32;
    const uint16_t *at = abf + (l & 31) * QFP_APITCH + 4 * (l >> 5);
    const uint16_t *wt = hmat + (4 * (l >> 5) + ((l & 15) >> 2)) * QFP_HPITCH + 16 * ((l >> 4) & 1) + 4 * (l & 3);
    // Eight rows at a time; the loads of the next eight (of this pass or of the wave's next one) are on their way
    // while the current eight are rotated: a pass would otherwise wait out four memory round trips.
    struct Rows8 {
        uint32_t raw[8], rc[8], rs[8];
    };
    auto load_rows = [&](Rows8 &r, const int pass, const int b8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int row = pass * 32 + b8 * 8 + u;
            const int rr = row < nrows ? row : nrows - 1;
            const int t = rr / p.n_heads;
            const int col = (rr - t * p.n_heads) * LIP_DIM + 2 * l;
            r.raw[u] = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint16_t *>(p.qpart) + (size_t)t * ncols + col);
            r.rc[u] = rope_coef(p.cos, t, l);
            r.rs[u] = rope_coef(p.sin, t, l);
        }
    };
    auto rotate_rows = [&](const Rows8 &r, const int b8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            float v0 = __uint_as_float(r.raw[u] << 16);        // the unsplit projection leaves its results de-quantised
            float v1 = __uint_as_float(r.raw[u] & 0xffff0000u);
            rope_pair(v0, v1, r.rc[u], r.rs[u], l);
            *reinterpret_cast<uint32_t *>(abf + (b8 * 8 + u) * QFP_APITCH + 2 * l) = pack_bf16x2(v0, v1);
        }
    };
    const int stride = nwg * QFP_WAVES;
    Rows8 ra, rb;
    if (wg * QFP_WAVES + w < npass) load_rows(ra, wg * QFP_WAVES + w, 0);
#pragma unroll 1
    for (int pass = wg * QFP_WAVES + w; pass < npass; pass += stride) {
        load_rows(rb, pass, 1);
        rotate_rows(ra, 0);
        load_rows(ra, pass, 2);
        rotate_rows(rb, 1);
        load_rows(rb, pass, 3);
        rotate_rows(ra, 2);
        if (pass + stride < npass) load_rows(ra, pass + stride, 0);
        rotate_rows(rb, 3);
        // the wave reads back what it wrote itself: LDS operations of a wave stay in order
        f32x16 c[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) c[cb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < LIP_DIM / 16; ++ks) {
            const u32x2 b0 = *reinterpret_cast<const u32x2 *>(at + 16 * ks);
            const u32x2 b1 = *reinterpret_cast<const u32x2 *>(at + 16 * ks + 8);
            const u32x4 bq = {b0[0], b0[1], b1[0], b1[1]};
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) {
                const s16x4 a0 = lds_read_tr16(wt + (16 * ks) * QFP_HPITCH + 32 * cb);
                const s16x4 a1 = lds_read_tr16(wt + (16 * ks + 8) * QFP_HPITCH + 32 * cb);
                const s16x8 a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                c[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, bq), c[cb], 0, 0, 0);
            }
        }
        // lane (row, half) holds channels 32*cb + 8*(r/4) + 4*half + r%4 of its row
        float amax = 0.f;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                c[cb][r] = bf16_round_f32(c[cb][r]);
                amax = fmaxf(amax, fabsf(c[cb][r]));
            }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(amax), __float_as_uint(amax), false, false);
            amax = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        float s = 0.f, deq = 0.f;
        if (amax > 0.f) {
            s = __fdiv_rn(127.0f, amax);
            deq = __fdiv_rn(1.0f, s);
        }
        uint8_t *orow = mine + (l & 31) * QFP_OPITCH + 4 * (l >> 5);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint32_t v = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) v |= (uint32_t)((int)rintf(__fmul_rn(c[cb][4 * g + j], s)) & 0xff) << (8 * j);
                *reinterpret_cast<uint32_t *>(orow + 32 * cb + 8 * g) = v;
            }
        const int row = pass * 32 + (l & 31);
        if (l < 32 && row < nrows) p.q_scale[row] = (uint16_t)(pack_f16x2(deq, 0.f) & 0xffffu);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int r = 8 * k + (l >> 3);
            const u32x4 v = *reinterpret_cast<const u32x4 *>(mine + r * QFP_OPITCH + 16 * (l & 7));
            if (pass * 32 + r < nrows) *reinterpret_cast<u32x4 *>(p.q_int8 + (size_t)(pass * 32 + r) * LIP_DIM + 16 * (l & 7)) = v;
        }
    }
}

// ---------------------------------------------------------------------------------- MLA prolog
constexpr int FIN_W_BYTES = MLAP_NOPE * 64 * 2;    // a wave's slice of w_uk[head]: 128 rows x 64 columns bf16
constexpr int MLAP_FIN_LDS = 4 * FIN_W_BYTES + MLAP_XTOK * MLAP_NOPE * 4 + MLAP_XTOK * MLAP_NOPE * 2;   // 71 680 bytes

// Workgroup (head, half of the 512 output columns, block of 8 tokens); wave w owns output columns
// colbase + 64w + l.
// The work of workgroup wg of the last launch (256 threads), in MLAP_FIN_LDS bytes of LDS at lds.
// workgroup barriers mlap_finish_body passes (every thread, unconditionally): a launch whose workgroups hold more
// than this body's 256 threads lets the surplus waves pass as many and leave
constexpr int MLAP_FIN_BARRIERS = 1;
__device__ __forceinline__ void mlap_finish_body(const MlapParams &p, const int wg, uint8_t *lds)
{
    uint8_t *wsl = lds;
    float(*arow)[MLAP_NOPE] = reinterpret_cast<float(*)[MLAP_NOPE]>(lds + 4 * FIN_W_BYTES);
    uint16_t(*abf)[MLAP_NOPE] = reinterpret_cast<uint16_t(*)[MLAP_NOPE]>(lds + 4 * FIN_W_BYTES + MLAP_XTOK * MLAP_NOPE * 4);   // the same values as bf16 (they are bf16-valued)
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int head = wg % p.n_heads;
    const int half = (wg / p.n_heads) & 1;
    const int t0 = (wg / p.n_heads / 2) * MLAP_XTOK;
    const int ncols = p.n_heads * MLAP_QHEAD;
    const int colbase = half * 256 + 64 * w;

    {   // this wave's slice: rows of 128 bytes, pitch 1024 bytes: 8 lanes per row, 8 rows per request
        const uint8_t *src = reinterpret_cast<const uint8_t *>(p.w_uk) + ((size_t)head * MLAP_NOPE + (l >> 3)) * (MLAP_KV * 2) +
                             colbase * 2 + 16 * (l & 7);
        const uint32_t dst = (uint32_t)(uintptr_t)(lds_byte_t *)(wsl + w * FIN_W_BYTES);
#pragma unroll 1
        for (int i = 0; i < MLAP_NOPE / 8; ++i) dma16(src + (size_t)i * 8 * MLAP_KV * 2, dst + 1024 * i);
    }
    // the head's query channels of tokens t0 + w and t0 + 4 + w: partial sums added, de-quantised, bf16
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int tl = 4 * u + w;
        const int t = t0 + tl;
        const int tt = t < p.T ? t : p.T - 1;
        const float ts = p.q_norm_scale[tt];
        // nope part: lane l -> channels 2l, 2l+1
        {
            const int col = head * MLAP_QHEAD + 2 * l;
            const f32x2 cs = *reinterpret_cast<const f32x2 *>(p.w_qb_scale + col);
            float av0, av1;
            q_value2(p.qpart, mlap_qsplits(p), p.T, tt, ncols, col, ts, cs[0], cs[1], av0, av1);
            const f32x2 av = {av0, av1};
            *reinterpret_cast<f32x2 *>(&arow[tl][2 * l]) = av;
            *reinterpret_cast<uint32_t *>(&abf[tl][2 * l]) = pack_bf16x2(av[0], av[1]);
        }
        // rope part (first half-workgroup only): lane l < 32 -> channels 2l, 2l+1 = rotation partners l, 32+l
        if (half == 0 && l < 32 && t < p.T) {
            const int col = head * MLAP_QHEAD + MLAP_NOPE + 2 * l;
            const f32x2 cs = *reinterpret_cast<const f32x2 *>(p.w_qb_scale + col);
            float v0, v1;
            q_value2(p.qpart, mlap_qsplits(p), p.T, t, ncols, col, ts, cs[0], cs[1], v0, v1);
            const float c0 = bf16_bits_to_f32(p.cos[(size_t)t * MLAP_ROPE + l]), c1 = bf16_bits_to_f32(p.cos[(size_t)t * MLAP_ROPE + 32 + l]);
            const float sn0 = bf16_bits_to_f32(p.sin[(size_t)t * MLAP_ROPE + l]), sn1 = bf16_bits_to_f32(p.sin[(size_t)t * MLAP_ROPE + 32 + l]);
            const float r0 = __builtin_fmaf(v0, c0, (-v1) * sn0);
            const float r1 = __builtin_fmaf(v1, c1, v0 * sn1);
            uint16_t *out = p.q_rope + ((size_t)t * p.n_heads + head) * MLAP_ROPE;
            out[l] = (uint16_t)(pack_bf16x2(r0, 0.f) & 0xffffu);
            out[32 + l] = (uint16_t)(pack_bf16x2(r1, 0.f) & 0xffffu);
        }
    }
    VM_WAIT(0);
    __syncthreads();                                   // (counted in MLAP_FIN_BARRIERS)

    if (!p.absorb_exact) {
        // On the matrix cores: C^T[col][token] = sum_i W^T[col][i] a^T[i][token], v_mfma_f32_32x32x16_bf16 with
        // A = the wave's slice of w_uk read transposed out of LDS (ds_read_b64_tr_b16: lane (col, half) gets rows
        // 16ks + 4*half + 0..3 and 16ks + 8 + 4*half + 0..3 of its column), B = the tokens' query values in the same
        // row order (lanes of tokens 8..31 repeat token 0; their results are not stored).  Two blocks of 32
        // columns, eight contraction steps.  Lane (token, half) then holds columns 8*(r/4) + 4*half + r%4 of a block.
        const uint16_t *wt = reinterpret_cast<const uint16_t *>(wsl + w * FIN_W_BYTES) +
                             (4 * (l >> 5) + ((l & 15) >> 2)) * 64 + 16 * ((l >> 4) & 1) + 4 * (l & 3);
        const int tok = (l & 31) < MLAP_XTOK ? (l & 31) : 0;
        const uint16_t *at = &abf[tok][4 * (l >> 5)];
        f32x16 c[2];
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) c[cb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < MLAP_NOPE / 16; ++ks) {
            const u32x2 b0 = *reinterpret_cast<const u32x2 *>(at + 16 * ks);
            const u32x2 b1 = *reinterpret_cast<const u32x2 *>(at + 16 * ks + 8);
            const u32x4 bq = {b0[0], b0[1], b1[0], b1[1]};
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const s16x4 a0 = lds_read_tr16(wt + (16 * ks) * 64 + 32 * cb);
                const s16x4 a1 = lds_read_tr16(wt + (16 * ks + 8) * 64 + 32 * cb);
                const s16x8 a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                c[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, bq), c[cb], 0, 0, 0);
            }
        }
        const int t = t0 + (l & 31);
        if ((l & 31) < MLAP_XTOK && t < p.T) {
            uint16_t *dst = p.q_nope + ((size_t)t * p.n_heads + head) * MLAP_KV + colbase + 4 * (l >> 5);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x2 v = {pack_bf16x2(c[cb][4 * q], c[cb][4 * q + 1]), pack_bf16x2(c[cb][4 * q + 2], c[cb][4 * q + 3])};
                    *reinterpret_cast<u32x2 *>(dst + 32 * cb + 8 * q) = v;
                }
        }
        return;
    }
    // out[t][colbase + 64w + l] = sum_i a[t][i] * w_uk[head][i][col], i ascending; 8 tokens at once.
    // Chunks of four rows are read one chunk ahead of the multiply-adds that consume them.
    const uint16_t *wl = reinterpret_cast<const uint16_t *>(wsl + w * FIN_W_BYTES) + l;
    float acc[MLAP_XTOK];
#pragma unroll
    for (int t = 0; t < MLAP_XTOK; ++t) acc[t] = 0.f;
    struct Chunk {
        f32x4 a[MLAP_XTOK];
        uint16_t w[4];
    };
    auto load = [&](Chunk &c, const int i) {
#pragma unroll
        for (int t = 0; t < MLAP_XTOK; ++t) c.a[t] = *reinterpret_cast<const f32x4 *>(&arow[t][i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) c.w[j] = wl[(i + j) * 64];
    };
    auto fma = [&](const Chunk &c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float wv = bf16_bits_to_f32(c.w[j]);
#pragma unroll
            for (int t = 0; t < MLAP_XTOK; ++t) acc[t] = __builtin_fmaf(c.a[t][j], wv, acc[t]);
        }
    };
    Chunk c0, c1;
    load(c0, 0);
#pragma unroll 1
    for (int i = 0; i < MLAP_NOPE; i += 8) {
        load(c1, i + 4);
        fma(c0);
        load(c0, i + 8 < MLAP_NOPE ? i + 8 : 0);
        fma(c1);
    }
#pragma unroll
    for (int t = 0; t < MLAP_XTOK; ++t)
        if (t0 + t < p.T)
            p.q_nope[((size_t)(t0 + t) * p.n_heads + head) * MLAP_KV + colbase + l] = (uint16_t)(pack_bf16x2(acc[t], 0.f) & 0xffffu);
}

// ------------------------------------------------------------------------ MLA prolog, prefill sizes
// The same last stage for MLAP_MFMA_MIN_TOKENS tokens and more with the absorb product on the matrix cores: one workgroup of eight
// waves per (head, run of `per` blocks of 32 tokens).  The head's whole w_uk (128 x 512 bf16, 128 KiB) is staged
// once, wave w keeping the slice of output columns 64w..64w+63 in the layout of the decode form; then per block:
// wave w moves the query channels of tokens 4w..4w+3 (de-quantised bf16 already: the projection is unsplit at these
// sizes) into one of two bf16 operand buffers and rotates and stores their rope part, the loads of the next block go out, one barrier, and
// 16 products per wave give 32 tokens x 64 columns.  A weight slice is read once per `per` blocks instead of once
// per 8 tokens; each output has the bits of the decode form (same products, same order).
constexpr int FINP_TOK = 32;
constexpr int FINP_WAVES = 8;
constexpr int FINP_APITCH = MLAP_NOPE + 8;   // elements between operand rows: 272 bytes, so that the 32 rows of an operand read spread over the banks
constexpr int FINP_SPITCH = 144;             // bytes between the rows of a wave's output staging area (8 tokens x 64 columns)
constexpr int FINP_STAGE = 8 * FINP_SPITCH;
constexpr int MLAP_FINP_LDS = FINP_WAVES * FIN_W_BYTES + 2 * FINP_TOK * FINP_APITCH * 2 + FINP_WAVES * FINP_STAGE;   // 157 696 bytes

struct FinRaw {
    uint32_t nope[4], rope[4];     // two bf16 values each: the unsplit projection leaves its results de-quantised
    uint16_t c0[4], c1[4], s0[4], s1[4];
};

__device__ __forceinline__ void mlap_finish_prefill_body(const MlapParams &p, const int wg, const int per, uint8_t *lds)
{
    uint8_t *wsl = lds;
    uint16_t(*abf)[FINP_TOK][FINP_APITCH] = reinterpret_cast<uint16_t(*)[FINP_TOK][FINP_APITCH]>(lds + FINP_WAVES * FIN_W_BYTES);
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int head = wg % p.n_heads;
    const int nblocks = (p.T + FINP_TOK - 1) / FINP_TOK;
    const int b0 = (wg / p.n_heads) * per;
    const int b1 = b0 + per < nblocks ? b0 + per : nblocks;
    const int ncols = p.n_heads * MLAP_QHEAD;
    const int colbase = 64 * w;

    {   // this wave's slice: rows of 128 bytes, pitch 1024 bytes: 8 lanes per row, 8 rows per request
        const uint8_t *src = reinterpret_cast<const uint8_t *>(p.w_uk) + ((size_t)head * MLAP_NOPE + (l >> 3)) * (MLAP_KV * 2) +
                             colbase * 2 + 16 * (l & 7);
        const uint32_t dst = (uint32_t)(uintptr_t)(lds_byte_t *)(wsl + w * FIN_W_BYTES);
#pragma unroll 1
        for (int i = 0; i < MLAP_NOPE / 8; ++i) dma16(src + (size_t)i * 8 * MLAP_KV * 2, dst + 1024 * i);
    }
    // lane l: nope channels 2l, 2l+1; lanes < 32: rope channels 2l, 2l+1 (= rotation partners l, 32+l)
    auto load = [&](FinRaw &r, const int blk) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = blk * FINP_TOK + 4 * w + u;
            const int tt = t < p.T ? t : p.T - 1;
            const uint16_t *row = reinterpret_cast<const uint16_t *>(p.qpart) + (size_t)tt * ncols + head * MLAP_QHEAD;
            r.nope[u] = *reinterpret_cast<const uint32_t *>(row + 2 * l);
            if (l < 32) {
                r.rope[u] = *reinterpret_cast<const uint32_t *>(row + MLAP_NOPE + 2 * l);
                r.c0[u] = p.cos[(size_t)tt * MLAP_ROPE + l];
                r.c1[u] = p.cos[(size_t)tt * MLAP_ROPE + 32 + l];
                r.s0[u] = p.sin[(size_t)tt * MLAP_ROPE + l];
                r.s1[u] = p.sin[(size_t)tt * MLAP_ROPE + 32 + l];
            }
        }
    };
    FinRaw raw;
    if (b0 < b1) load(raw, b0);
    VM_WAIT(0);

    const uint16_t *wt = reinterpret_cast<const uint16_t *>(wsl + w * FIN_W_BYTES) +
                         (4 * (l >> 5) + ((l & 15) >> 2)) * 64 + 16 * ((l >> 4) & 1) + 4 * (l & 3);
#pragma unroll 1
    for (int blk = b0; blk < b1; ++blk) {
        const int buf = (blk - b0) & 1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int tl = 4 * w + u;
            const int t = blk * FINP_TOK + tl;
            *reinterpret_cast<uint32_t *>(&abf[buf][tl][2 * l]) = raw.nope[u];
            if (l < 32 && t < p.T) {
                const float v0 = __uint_as_float(raw.rope[u] << 16);
                const float v1 = __uint_as_float(raw.rope[u] & 0xffff0000u);
                const float r0 = __builtin_fmaf(v0, bf16_bits_to_f32(raw.c0[u]), (-v1) * bf16_bits_to_f32(raw.s0[u]));
                const float r1 = __builtin_fmaf(v1, bf16_bits_to_f32(raw.c1[u]), v0 * bf16_bits_to_f32(raw.s1[u]));
                uint16_t *out = p.q_rope + ((size_t)t * p.n_heads + head) * MLAP_ROPE;
                out[l] = (uint16_t)(pack_bf16x2(r0, 0.f) & 0xffffu);
                out[32 + l] = (uint16_t)(pack_bf16x2(r1, 0.f) & 0xffffu);
            }
        }
        if (blk + 1 < b1) load(raw, blk + 1);
        __syncthreads();                               // this block's operands are complete; the other buffer is free

        const uint16_t *at = &abf[buf][l & 31][4 * (l >> 5)];
        f32x16 c[2];
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) c[cb][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < MLAP_NOPE / 16; ++ks) {
            const u32x2 bq0 = *reinterpret_cast<const u32x2 *>(at + 16 * ks);
            const u32x2 bq1 = *reinterpret_cast<const u32x2 *>(at + 16 * ks + 8);
            const u32x4 bq = {bq0[0], bq0[1], bq1[0], bq1[1]};
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const s16x4 a0 = lds_read_tr16(wt + (16 * ks) * 64 + 32 * cb);
                const s16x4 a1 = lds_read_tr16(wt + (16 * ks + 8) * 64 + 32 * cb);
                const s16x8 a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                c[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, bq), c[cb], 0, 0, 0);
            }
        }
        // Lane (token, half) holds 8-byte fragments of its token's row; they leave through the wave's staging area,
        // eight tokens at a time, as whole 128-byte rows (16 bytes per lane) -- scattered fragments cost the memory
        // side several times their bytes.
        uint8_t *stg = lds + FINP_WAVES * FIN_W_BYTES + 2 * FINP_TOK * FINP_APITCH * 2 + w * FINP_STAGE;
#pragma unroll
        for (int qt = 0; qt < 4; ++qt) {
            if (((l & 31) >> 3) == qt) {
                uint8_t *row = stg + (l & 7) * FINP_SPITCH + 8 * (l >> 5);
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const u32x2 v = {pack_bf16x2(c[cb][4 * q], c[cb][4 * q + 1]), pack_bf16x2(c[cb][4 * q + 2], c[cb][4 * q + 3])};
                        *reinterpret_cast<u32x2 *>(row + 64 * cb + 16 * q) = v;
                    }
            }
            const u32x4 v = *reinterpret_cast<const u32x4 *>(stg + (l >> 3) * FINP_SPITCH + 16 * (l & 7));
            const int t = blk * FINP_TOK + 8 * qt + (l >> 3);
            if (t < p.T) *reinterpret_cast<u32x4 *>(p.q_nope + ((size_t)t * p.n_heads + head) * MLAP_KV + colbase + 8 * (l & 7)) = v;
        }
    }
}

}  // namespace
}  // namespace pto
