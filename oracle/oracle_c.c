/*
 * Scalar C statement of the two CPU goldens of the quantized DeepSeek-V3.2
 * sparse-attention path.  TEST INFRASTRUCTURE ONLY: linked by nothing in the
 * shipped package; loaded with ctypes by tests/, by the smoke check and by the
 * cpu_baseline leg of the benchmark.
 *
 * It is written independently of the torch statement in sfa_oracle.py /
 * li_oracle.py (own bf16 / fp16 rounding with integer arithmetic, explicit
 * loops, qsort for the select) so that agreement between the two is evidence,
 * not a tautology.
 *
 * Reference (paths relative to the reference tree):
 *   oracle_sfa_quant   examples/models/deepseek_v32_exp/
 *                      deepseekv32_sparse_flash_attention_quant.py:169-254
 *                      (single pass) and :49-166 (online, s2_tile > 0)
 *   oracle_li_decode   examples/models/deepseek_v32_exp/
 *                      deepseekv32_lightning_indexer_quant.py:184-269
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off -fopenmp).
 * -ffp-contract=off matters: the indexer's head sum is defined as a rounded
 * multiply followed by a rounded add.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---------- scalar format helpers (integer arithmetic only) ---------- */

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return u32_as_f32(((uint32_t)h) << 16); }

/* round-to-nearest-even fp32 -> bf16 (finite inputs; NaN kept quiet) */
static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u = f32_as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float fp16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u32_as_f32(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return u32_as_f32(sign | 0x7f800000u | (man << 13));
    return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even fp32 -> fp16, all finite inputs incl. subnormal results */
static inline uint16_t f32_to_fp16(float f)
{
    uint32_t u = f32_as_u32(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);       /* >= 65536 -> inf */
    if (a >= 0x38800000u) {                                         /* normal fp16 range */
        uint32_t v = a - 0x38000000u;                               /* rebias exponent by 112 */
        uint32_t lsb = (v >> 13) & 1u;
        v += 0xfffu + lsb;
        v >>= 13;
        /* 65520 <= x < 65536 rounds up into 0x7c00 = inf, as IEEE requires */
        return (uint16_t)(sign | v);
    }
    if (a < 0x33000000u) return sign;                               /* < 2^-25 -> 0 */
    /* subnormal result: value = m * 2^-24 with m = round(a_val * 2^24) */
    uint32_t e = a >> 23;                                           /* 102 .. 112 */
    uint32_t m = (a & 0x7fffffu) | 0x800000u;                       /* 24-bit significand */
    uint32_t shift = 126u - e;                                      /* 14 .. 24 */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

static int g_threads = 0;
void oracle_set_threads(int n) { g_threads = n; }
int oracle_get_threads(void)
{
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

/* exported so the Python tests can pin the rounding helpers themselves */
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
uint16_t oracle_f32_to_fp16(float f) { return f32_to_fp16(f); }
float oracle_fp16_to_f32(uint16_t h) { return fp16_to_f32(h); }

/* ---------- sparse flash attention ---------- */

static inline int64_t phys_row(const int32_t *bt_row, int32_t idx, int bs)
{
    return (int64_t)bt_row[idx / bs] * bs + idx % bs;
}

/*
 * q_nope [T*N, DN] bf16, q_rope [T*N, DR] bf16, kn [rows, DN] int8, kr [rows, DR] bf16,
 * kn_scales [rows, 4] fp32, topk_idx [T, topk] int32, block_table [B, max_blocks] int32,
 * act_seq [B] int32, out [T*N, DN] bf16.  s2_tile == 0: single-pass golden; > 0: online.
 * Rows with cur_seq == 0 are written as zeros.
 */
int oracle_sfa_quant(const uint16_t *q_nope, const uint16_t *q_rope, const int8_t *kn, const uint16_t *kr,
                     const float *kn_scales, const int32_t *topk_idx, const int32_t *block_table,
                     const int32_t *act_seq, uint16_t *out, int B, int S1, int N, int DN, int DR, int topk,
                     int block_size, int max_blocks, float scalar, int s2_tile)
{
    const int D = DN + DR;
    const int G = DN / 4;
    int rc = 0;
    for (int b = 0; b < B; b++) {
        for (int s = 0; s < S1; s++) {
            int t = b * S1 + s;
            int cur = act_seq[b] - S1 + 1 + s;
            if (cur < 0) cur = 0;
            if (cur > topk) cur = topk;
            uint16_t *o_t = out + (size_t)t * N * DN;
            if (cur == 0) { memset(o_t, 0, (size_t)N * DN * 2); continue; }
            float *kj = (float *)malloc((size_t)cur * D * sizeof(float));
            if (!kj) return -1;
            for (int j = 0; j < cur; j++) {
                int64_t r = phys_row(block_table + (size_t)b * max_blocks, topk_idx[(size_t)t * topk + j], block_size);
                for (int c = 0; c < DN; c++) {
                    float v = (float)kn[r * DN + c] * kn_scales[r * 4 + c / G];
                    kj[(size_t)j * D + c] = bf16_to_f32(f32_to_bf16(v));
                }
                for (int c = 0; c < DR; c++) kj[(size_t)j * D + DN + c] = bf16_to_f32(kr[r * DR + c]);
            }
            int tile = s2_tile > 0 ? s2_tile : cur;
#pragma omp parallel for schedule(dynamic, 1) num_threads(oracle_get_threads())
            for (int h = 0; h < N; h++) {
                float *qf = (float *)malloc(sizeof(float) * D);
                float *sc = (float *)malloc(sizeof(float) * tile);
                float *acc = (float *)malloc(sizeof(float) * DN);
                float *part = (float *)malloc(sizeof(float) * DN);
                for (int c = 0; c < DN; c++) qf[c] = bf16_to_f32(q_nope[((size_t)t * N + h) * DN + c]);
                for (int c = 0; c < DR; c++) qf[DN + c] = bf16_to_f32(q_rope[((size_t)t * N + h) * DR + c]);
                float m_run = 0.f, l_run = 0.f;
                for (int lo = 0, it = 0; lo < cur; lo += tile, it++) {
                    int n = cur - lo < tile ? cur - lo : tile;
                    float m_t = -INFINITY;
                    for (int j = 0; j < n; j++) {
                        const float *kr_ = kj + (size_t)(lo + j) * D;
                        float a = 0.f;
                        for (int c = 0; c < D; c++) a += qf[c] * kr_[c];
                        a *= scalar;
                        sc[j] = a;
                        if (a > m_t) m_t = a;
                    }
                    float l_t = 0.f;
                    for (int j = 0; j < n; j++) { sc[j] = expf(sc[j] - m_t); l_t += sc[j]; }
                    for (int c = 0; c < DN; c++) part[c] = 0.f;
                    for (int j = 0; j < n; j++) {
                        float p = s2_tile > 0 ? sc[j] : sc[j] / l_t;
                        p = bf16_to_f32(f32_to_bf16(p));
                        const float *v = kj + (size_t)(lo + j) * D;
                        for (int c = 0; c < DN; c++) part[c] += p * v[c];
                    }
                    if (it == 0) {
                        memcpy(acc, part, sizeof(float) * DN);
                        m_run = m_t; l_run = l_t;
                    } else {
                        float m_new = m_run > m_t ? m_run : m_t;
                        float a_old = expf(m_run - m_new), a_new = expf(m_t - m_new);
                        l_run = a_old * l_run + a_new * l_t;
                        for (int c = 0; c < DN; c++) acc[c] = acc[c] * a_old + part[c] * a_new;
                        m_run = m_new;
                    }
                }
                for (int c = 0; c < DN; c++) {
                    float v = s2_tile > 0 ? acc[c] / l_run : acc[c];
                    o_t[(size_t)h * DN + c] = f32_to_bf16(v);
                }
                free(qf); free(sc); free(acc); free(part);
            }
            free(kj);
        }
    }
    return rc;
}

/* ---------- lightning indexer ---------- */

enum { ORACLE_FP16 = 0, ORACLE_FP32 = 1, ORACLE_BF16 = 2 };

static inline float load_scalar(const void *p, size_t i, int dt)
{
    switch (dt) {
    case ORACLE_FP16: return fp16_to_f32(((const uint16_t *)p)[i]);
    case ORACLE_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

typedef struct { float s; int32_t i; } pair_t;

static int cmp_pair(const void *a, const void *b)
{
    const pair_t *x = (const pair_t *)a, *y = (const pair_t *)b;
    if (x->s > y->s) return -1;          /* -0.0 and +0.0 compare equal here */
    if (x->s < y->s) return 1;
    return (x->i > y->i) - (x->i < y->i);
}

/*
 * q [T,H,D] int8; q_scale [T,H] (q_dt); kcache [NB*bs, D] int8; k_scale [NB*bs] (k_dt);
 * weight [T,H] (w_dt); act_seq [B]; block_table [B,max_blocks]; topk_res [T,k] int32;
 * scores_out: optional [T, score_stride] fp32 (may be NULL).
 */
int oracle_li_decode(const int8_t *q, const void *q_scale, int q_dt, const int8_t *kcache, const void *k_scale,
                     int k_dt, const void *weight, int w_dt, const int32_t *act_seq, const int32_t *block_table,
                     int32_t *topk_res, float *scores_out, int64_t score_stride, int B, int S1, int H, int D,
                     int block_size, int max_blocks, int k)
{
    int T = B * S1;
    int rc = 0;
#pragma omp parallel for schedule(dynamic, 1) num_threads(oracle_get_threads())
    for (int t = 0; t < T; t++) {
        int b = t / S1, s = t % S1;
        int cur = act_seq[b];
        if (cur < 0) cur = 0;
        float *wsc = (float *)malloc(sizeof(float) * H);
        float *score = (float *)malloc(sizeof(float) * (cur > 0 ? cur : 1));
        for (int h = 0; h < H; h++) {
            float qs = load_scalar(q_scale, (size_t)t * H + h, q_dt);
            float w = load_scalar(weight, (size_t)t * H + h, w_dt);
            float p = qs * w;                                   /* one fp32 rounding */
            if (q_dt == ORACLE_FP16 && w_dt == ORACLE_FP16) p = fp16_to_f32(f32_to_fp16(p));
            wsc[h] = p;
        }
        const int8_t *qt = q + (size_t)t * H * D;
        for (int j = 0; j < cur; j++) {
            int64_t r = phys_row(block_table + (size_t)b * max_blocks, j, block_size);
            const int8_t *kr_ = kcache + r * D;
            float acc = 0.f;
            for (int h = 0; h < H; h++) {
                int32_t dot = 0;
                for (int d = 0; d < D; d++) dot += (int32_t)qt[h * D + d] * (int32_t)kr_[d];
                float rl = dot > 0 ? (float)dot : 0.f;
                float x = fp16_to_f32(f32_to_fp16(rl * (1.0f / 2048.0f)));
                float prod = wsc[h] * x;
                acc = acc + prod;
            }
            score[j] = acc * load_scalar(k_scale, (size_t)r, k_dt);
        }
        if (scores_out) memcpy(scores_out + (size_t)t * score_stride, score, sizeof(float) * cur);
        int eff = cur - (S1 - 1 - s);
        if (eff < 0) eff = 0;
        pair_t *pr = (pair_t *)malloc(sizeof(pair_t) * (eff > 0 ? eff : 1));
        for (int j = 0; j < eff; j++) { pr[j].s = score[j]; pr[j].i = j; }
        qsort(pr, eff, sizeof(pair_t), cmp_pair);
        for (int j = 0; j < k; j++) topk_res[(size_t)t * k + j] = j < eff ? pr[j].i : -1;
        free(pr); free(score); free(wsc);
    }
    return rc;
}
