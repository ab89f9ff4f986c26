// Launch parameters of the MLA prolog kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

constexpr int MLAP_NOPE = 128;       // query channels per head that meet w_uk
constexpr int MLAP_ROPE = 64;        // rotated channels per head and of the key
constexpr int MLAP_KV = 512;         // latent width
constexpr int MLAP_QHEAD = MLAP_NOPE + MLAP_ROPE;
constexpr int MLAP_XBLOCK = 64;      // block length of the fixed-order sums over the hidden axis
constexpr int MLAP_XGROUP = 8;       // block sums per group (one workgroup of the first kernel)
constexpr int MLAP_MAX_XGROUPS = 32; // h <= 32 * 8 * 64 = 16384
constexpr int MLAP_MAX_QLORA = 1536;
constexpr int QPROJ_KSPLIT_HOST = 4; // partial sums of the int8 projection (prolog_common.h: QPROJ_KSPLIT)
constexpr int MLAP_XTOK = 8;         // tokens per job of the first and of the last kernel
constexpr int MLAP_MFMA_MIN_TOKENS = 9;    // from here on the stages take their prefill forms unless absorb_exact: the first launch
                                           // sums on the matrix cores, the projection runs unsplit, the last stage walks token blocks
                                           // per head (the decode forms work on 8 tokens at a time and their cost grows with every
                                           // 8 tokens; those forms cost the same from 9 to 128 tokens, about what 8 tokens cost here)
constexpr int MLAP_UNSPLIT_MIN_TOKENS = 64;   // with absorb_exact the projection still runs unsplit from here on
// ranges of the hidden axis (partial sums per token) of that form, at most.  With a single token tile the sixteen
// matrix-core slabs x 14 ranges and the rope columns' 32 workgroups are one workgroup per compute unit of an
// MI355X, every one requesting weights from the start (8 ranges: 32 tokens 44.6 us per pass, 14: 40.9, 20 or 28: 43.3)
constexpr int MLAP_XM_MAX_SPLITS = 14;

// rows [T, q_lora + 576] of partial sums over the hidden axis the workspace holds: the group sums of the
// fixed-order form, or the ranges of the matrix-core form where that may run
inline int mlap_xpart_rows(const int h, const int T)
{
    const int nblk = h / MLAP_XBLOCK;
    const int groups = (nblk + MLAP_XGROUP - 1) / MLAP_XGROUP;
    const int splits = T >= MLAP_MFMA_MIN_TOKENS ? (nblk < MLAP_XM_MAX_SPLITS ? nblk : MLAP_XM_MAX_SPLITS) : 0;
    return groups > splits ? groups : splits;
}

struct MlapParams {
    const uint16_t *x;            // [T, h] bf16
    const uint16_t *w_dq;         // [h, q_lora] bf16
    const int8_t *w_uqqr;         // [q_lora, n_heads*192] int8
    const float *w_qb_scale;      // [n_heads*192]
    const uint16_t *w_uk;         // [n_heads, 128, 512] bf16
    const uint16_t *w_dkvkr;      // [h, 576] bf16
    const uint16_t *gamma_cq;     // [q_lora] bf16
    const uint16_t *gamma_ckv;    // [512] bf16
    const uint16_t *cos;          // [T, 64] bf16
    const uint16_t *sin;          // [T, 64] bf16
    const long long *cache_index; // [T]
    int8_t *kv_cache;             // [cache_rows, 512]
    uint16_t *kr_cache;           // [cache_rows, 64] bf16
    float *k_scale_cache;         // [cache_rows, 4]
    int8_t *q_norm;               // [T, q_lora]         written, then read by the projection
    float *q_norm_scale;          // [T]
    uint16_t *q_nope;             // [T, n_heads, 512] bf16
    uint16_t *q_rope;             // [T, n_heads, 64] bf16
    float *xpart;                 // workspace [ceil(h/512), T, q_lora + 576]
    int32_t *qpart;               // workspace [4, T, n_heads*192]
    long long cache_rows;
    int T, h, q_lora, n_heads;
    float eps_cq, eps_ckv;
    int absorb_exact;             // 1: the product with w_uk as fixed-order fp32 sums (bit-reproducible against the
                                  // sequential statement); 0: on the matrix cores (bf16 x bf16 exact, fp32 sums in the
                                  // cores' own order: differs in the last bit of some results), and from
                                  // MLAP_MFMA_MIN_TOKENS tokens on the sums over the hidden axis as well
};

// Work of the lightning-indexer prolog that the decode form's launches can carry along (the fused operator): its
// sums over the hidden axis have the same fixed order as this prolog's and its int8 projection reads the same
// q_norm, so wk rides as one more column slab of the first launch, w_proj shares the slab of w_dkv_kr's 64 rope
// columns, and the projection's jobs follow this prolog's in the third launch.
struct MlapRider {
    const uint16_t *wk;      // [h, 128] bf16
    const uint16_t *w_proj;  // [h, 64] bf16
    float *xpart;            // group sums [ceil(h/512), T, 192]: wk's columns, then w_proj's
    const int8_t *w_qb;      // [q_lora, 128 * q_slabs] int8
    int32_t *qpart;          // partial sums [4, T, 128 * q_slabs]
    int q_slabs;
};

// the stages' prefill forms (matrix-core sums over the hidden axis, last stage per head and run of token blocks)
__host__ __device__ inline bool mlap_prefill_forms(const MlapParams &p) { return p.T >= MLAP_MFMA_MIN_TOKENS && !p.absorb_exact; }
// partial sums per output the int8 projection leaves: 1 = unsplit (de-quantised bf16), else QPROJ_KSPLIT_HOST int32 partials
__host__ __device__ inline int mlap_qsplits(const MlapParams &p)
{
    return (mlap_prefill_forms(p) || p.T >= MLAP_UNSPLIT_MIN_TOKENS) ? 1 : QPROJ_KSPLIT_HOST;
}
// whether the launches of `p` take a rider at all: the decode forms only
inline bool mlap_takes_rider(const MlapParams &p) { return !mlap_prefill_forms(p) && mlap_qsplits(p) != 1; }

hipError_t mlap_launch(const MlapParams &p, hipStream_t stream);
// all launches but the last, and the number of workgroups of the last (for the fused operator's last launch)
// lip_rider (prefill forms below 64 tokens only): the indexer prolog whose first launch's jobs -- fixed-order sums
// over the hidden axis, split int8 projection -- ride in this operator's first and third launch
struct LipParams;
hipError_t mlap_launch_front(const MlapParams &p, hipStream_t stream, const MlapRider *rider = nullptr, const LipParams *lip_rider = nullptr);
// whether the launches of `p` take such a rider
inline bool mlap_takes_lip_rider(const MlapParams &p) { return mlap_prefill_forms(p) && p.T < 64; }
int mlap_finish_wgs(const MlapParams &p);
// the last launch alone; at prefill sizes (mlap_finish_is_prefill) it has a form of its own that the fused operator
// launches beside, not inside, its own last launch
hipError_t mlap_launch_finish(const MlapParams &p, hipStream_t stream);
bool mlap_finish_is_prefill(const MlapParams &p);
// blocks of 32 tokens per workgroup and workgroups of that form's launch
void mlap_finish_prefill_shape(const MlapParams &p, int &per, int &wgs);

}  // namespace pto
