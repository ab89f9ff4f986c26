// Launch parameters of the lightning-indexer prolog kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

constexpr int LIP_DIM = 128;        // channels per indexer head
constexpr int LIP_ROPE = 64;        // leading channels that are rotated
constexpr int LIP_KSPLIT = 4;       // workgroups that share the reduction axis of the query projection (= QPROJ_KSPLIT of the shared job code)
constexpr int LIP_XBLOCK = 64;      // block length of the fixed-order sums over the hidden axis
constexpr int LIP_XGROUP = 8;       // block sums per group of the second level of those sums
constexpr int LIP_MAX_XGROUPS = 24; // groups the finishing kernel keeps in LDS: h <= 24 * 8 * 64 = 12288
constexpr int LIP_XCOLS = 192;      // columns of one partial row: 128 key channels, then up to 64 head weights
constexpr int LIP_MAX_HEADS = 64;
constexpr int LIP_MAX_QLORA = 1536; // a wave keeps the requests of its eighth of w_qb (q_lora_rank/8 rows) and of its token rows in flight at once (at most 63)

struct LipParams {
    const uint16_t *x;           // [T, h] bf16
    const int8_t *q_norm;        // [T, q_lora]
    const float *q_norm_scale;   // [T]
    const int8_t *w_qb;          // [q_lora, n_heads*128]
    const float *w_qb_scale;     // [n_heads*128]
    const uint16_t *wk;          // [h, 128] bf16
    const uint16_t *w_proj;      // [h, n_heads] bf16
    const uint16_t *gamma;       // [128] bf16
    const uint16_t *beta;        // [128] bf16
    const uint16_t *cos;         // [T, 64] bf16
    const uint16_t *sin;         // [T, 64] bf16
    const uint16_t *hq;          // [128, 128] bf16
    const uint16_t *hk;          // [128, 128] bf16
    int8_t *k_cache;             // [cache_rows, 128]
    uint16_t *k_cache_scale;     // [cache_rows] fp16
    const long long *k_cache_index;  // [T]
    int8_t *q_int8;              // [T, n_heads, 128]
    uint16_t *q_scale;           // [T, n_heads] fp16
    uint16_t *weights;           // [T, n_heads] fp16
    int32_t *qpart;              // workspace [LIP_KSPLIT, T, n_heads*128]
    float *xpart;                // workspace [h/64, T, LIP_XCOLS]
    long long cache_rows;
    int T, h, q_lora, n_heads;
    float eps, w_mul0, w_mul1;   // weights = fp16((bf16(x.w_proj) * w_mul0) * w_mul1)
    int sum_mode;                // LIP_SUMS_*
    int x_in_groups;             // 1: xpart already holds one row per group of eight blocks, left there by another
                                 // operator's launch (the fused prolog at decode sizes); set by that launcher only
};

// How the fp32 sums are taken from LIP_MFMA_MIN_TOKENS tokens on (below that every sum has its fixed order):
constexpr int LIP_SUMS_DEFAULT = 0;        // the query rows' Hadamard sums on the matrix cores, everything else fixed-order
constexpr int LIP_SUMS_EXACT = 1;          // every sum in its fixed order
constexpr int LIP_SUMS_MATRIX_CORES = 2;   // the sums over the hidden axis on the matrix cores as well
constexpr int LIP_MFMA_MIN_TOKENS = 64;
constexpr int LIP_XM_MAX_SPLITS = 16;    // ranges of the hidden axis (partial sums per token) of the matrix-core form, at most

__host__ __device__ inline bool lip_q_on_matrix_cores(const LipParams &p)
{
    return p.T >= LIP_MFMA_MIN_TOKENS && p.sum_mode != LIP_SUMS_EXACT;
}
// the hidden-axis form needs w_proj rows made of whole 16-byte pieces
__host__ __device__ inline bool lip_x_on_matrix_cores(const LipParams &p)
{
    return p.T >= LIP_MFMA_MIN_TOKENS && p.sum_mode == LIP_SUMS_MATRIX_CORES && p.n_heads % 8 == 0;
}
// the fixed-order sums over the hidden axis at prefill sizes leave one row per group of eight blocks (the group sums)
// instead of one per block; the staging of that form needs w_proj rows of a power of two of 16-byte pieces
__host__ __device__ inline bool lip_x_group_rows(const LipParams &p)
{
    const int wb = p.n_heads * 2;
    if (p.x_in_groups) return true;
    return p.T >= LIP_MFMA_MIN_TOKENS && !lip_x_on_matrix_cores(p) && wb >= 16 && (wb & (wb - 1)) == 0;
}
// partial rows [T, LIP_XCOLS] the first launch leaves per token: the blocks of 64 of the fixed-order form, or the
// ranges of the matrix-core form (enough of them for about 512 workgroups of 128 tokens x 128 columns: two per compute unit)
__host__ __device__ inline int lip_xrows(const LipParams &p)
{
    const int nblk = p.h / LIP_XBLOCK;
    if (lip_x_group_rows(p)) return (nblk + LIP_XGROUP - 1) / LIP_XGROUP;
    if (!lip_x_on_matrix_cores(p)) return nblk;
    int s = 256 / ((p.T + 127) / 128);
    s = s < 1 ? 1 : s;
    s = s > LIP_XM_MAX_SPLITS ? LIP_XM_MAX_SPLITS : s;
    return s > nblk ? nblk : s;
}

hipError_t lip_launch(const LipParams &p, hipStream_t stream);
// the first launch alone, and the number of query-row workgroups of the second (for the fused operator's last launch)
hipError_t lip_launch_linear(const LipParams &p, hipStream_t stream);
int lip_finish_query_wgs(const LipParams &p);
hipError_t lip_launch_finish(const LipParams &p, hipStream_t stream);   // the second launch alone

}  // namespace pto
