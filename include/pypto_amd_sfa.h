/*
 * C ABI of the MI355X (gfx950) implementation of the quantized DeepSeek-V3.2
 * sparse-attention path: the lightning indexer (score + top-k select) and the
 * sparse flash attention that consumes its indices.
 *
 * Plain pointers and sizes only; every pointer is a DEVICE pointer unless stated
 * otherwise.  The caller owns all memory, including outputs and the workspace.
 * Launches are asynchronous on the HIP stream passed in (a hipStream_t cast to
 * void*; NULL = the default stream); nothing here synchronises.
 *
 * Return value: 0 on success, a negative PTO_E_* code otherwise;
 * pto_last_error() returns a thread-local, NUL-terminated description of the
 * last failure on the calling thread.
 *
 * What each entry point replaces in the reference (paths relative to the
 * reference tree):
 *
 *   pto_sfa_quant_launch
 *       the device execution of sparse_flash_attention_quant_d / _p
 *       (examples/models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:437-476,
 *       499-538), i.e. what python/pypto/runtime.py:153 dispatches through
 *       ExportedOperatorDeviceLaunchOnceWithDeviceTensorData
 *       (framework/src/machine/runtime/device_launcher_binding.h:204-209).
 *   pto_sa_antiquant_launch
 *       the device execution of sparse_attention_antiquant_d / _p
 *       (examples/models/deepseek_v32_exp/sparse_attention_antiquant_impl.py:263-300,
 *       322-359), same dispatch point: the same attention over the packed cache
 *       layout (one 656-byte row per key).
 *   pto_li_decode_launch
 *       the device execution of lightning_indexer_decode
 *       (examples/models/deepseek_v32_exp/lightning_indexer_quant_impl.py:315-346),
 *       same dispatch point.
 *   pto_li_prolog_quant_launch
 *       the device execution of lightning_indexer_prolog_quant
 *       (examples/models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:507-562),
 *       same dispatch point: the projection stage that produces the indexer's
 *       int8 query, per-head weights and the new int8 key rows of the paged cache.
 *   pto_mla_prolog_quant_launch
 *       the device execution of mla_prolog_quant_d / _p
 *       (examples/models/deepseek_v32_exp/mla_prolog_quant_impl.py:710-869), same
 *       dispatch point: the projection stage that produces the attention's query
 *       (absorbed nope part and rope part), the int8 query latent the indexer prolog
 *       consumes, and the new rows of the latent / rope / scale caches.
 *   pto_*_workspace_bytes
 *       the workspace query the reference runtime performs before a launch
 *       (python/pypto/runtime.py:151-152, GetWorkSpaceSize).
 */
#ifndef PYPTO_AMD_SFA_H
#define PYPTO_AMD_SFA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTO_OK 0
#define PTO_E_INVALID_ARG (-1) /* NULL pointer, unsupported shape or dtype code      */
#define PTO_E_WORKSPACE (-2)   /* workspace missing or smaller than *_workspace_bytes */
#define PTO_E_LAUNCH (-3)      /* the HIP runtime refused the launch                  */
#define PTO_E_NO_DEVICE (-4)   /* no gfx950 device / code object not loadable        */

/* element types of the indexer's scale and weight tensors */
#define PTO_DT_FP16 0
#define PTO_DT_FP32 1
#define PTO_DT_BF16 2

/*
 * Sparse flash attention over the paged int8 latent-KV cache.
 * Tensor names, shapes and layouts are those of sparse_flash_attention_quant_d
 * (sparse_flash_attention_quant_impl.py:45-85 in the reference example):
 *
 *   query_nope    [b*s1*nq, 512]            bf16
 *   query_rope    [b*s1*nq, 64]             bf16
 *   key_nope_2d   [kv_rows, 512]            int8    kv_rows = block_num*block_size
 *   key_rope_2d   [kv_rows, 64]             bf16
 *   k_nope_scales [kv_rows, 4]              fp32    one scale per 128 channels
 *   topk_indices  [b*s1, n_kv*topk]         int32   logical key positions
 *   block_table   [b, max_blocknum_perbatch] int32  logical block -> physical block
 *   kv_act_seqs   [b]                        int32
 *   attention_out [b, s1, nq, 512]          bf16    written in place
 *
 * Query row (bi, si) attends to the first
 *   cur_seq = min(max(kv_act_seqs[bi] - s1 + 1 + si, 0), topk)
 * entries of its index row; rows with cur_seq == 0 are written as zeros.
 * Indices that would address memory outside [0, kv_rows) are clamped into it
 * (the reference reads unchecked); their contribution is unspecified.
 *
 * Constraints: n_kv == 1, topk >= 1, block_size >= 1, nq >= 1.
 * Alignment: query, cache, output and workspace pointers 16 bytes (a contiguous
 * torch view with a storage offset may not be), the int32 tensors 4 bytes.
 * num_splits: how many workgroups share one query row's keys (0 = the count
 * that fills the device's compute units in one round of workgroups, or the
 * nearest count below that when the batch does not divide them).  When a row is split, each split's result
 * travels as fp16 normalised by the split's own row sum: de-quantised cache
 * values must stay below 65504 in magnitude (always true of int8 * scale for
 * sane scales; for the bf16 cache of pto_sfa_bf16kv_launch larger values give
 * inf/NaN unless num_splits == 1).
 */
typedef struct PtoSfaQuantArgs {
    const void *query_nope;
    const void *query_rope;
    const void *key_nope_2d;
    const void *key_rope_2d;
    const void *k_nope_scales;
    const int32_t *topk_indices;
    const int32_t *block_table;
    const int32_t *kv_act_seqs;
    void *attention_out;
    void *workspace;
    size_t workspace_bytes;
    int64_t b;
    int64_t s1;
    int64_t nq;
    int64_t n_kv;
    int64_t topk;
    int64_t block_size;
    int64_t max_blocknum_perbatch;
    int64_t kv_rows;
    float softmax_scale;
    int32_t num_splits;
} PtoSfaQuantArgs;

int pto_sfa_quant_workspace_bytes(const PtoSfaQuantArgs *args, size_t *bytes);
int pto_sfa_quant_launch(const PtoSfaQuantArgs *args, void *hip_stream);

/*
 * pto_sfa_quant_launch for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc): it has no
 * counterpart in the reference.  The partial results of the key splits go to an
 * array built into the library (PTO_SFA_STATIC_SCRATCH_BYTES per GPU, held until
 * the process ends) instead of a workspace; args->workspace and workspace_bytes
 * are ignored.  Nothing is allocated or freed; the first call on a device looks
 * the array's device address up.  With num_splits = 0 the library takes the best
 * split count whose partial results fit the array (the decode shapes this library
 * is benchmarked on fit as they are: 32 rows x 8 splits and 128 rows x 2 splits of
 * 128 heads take 33.8 MB).  An explicit num_splits, or a top-k past what one
 * workgroup holds, whose splits need more than the array holds is refused with
 * PTO_E_WORKSPACE.
 * All calls on one GPU share the array: calls whose execution may overlap (two
 * streams, two threads) race on it and must use pto_sfa_quant_launch with
 * workspaces of their own instead.  Nothing in the array has to be cleared
 * between calls: every split writes its partial before it is read.
 */
#define PTO_SFA_STATIC_SCRATCH_BYTES ((size_t)40 << 20)
int pto_sfa_quant_launch_static(const PtoSfaQuantArgs *args, void *hip_stream);

/*
 * The non-quantized branch of the same operator (key_nope_2d not int8,
 * sparse_flash_attention_quant_impl.py:149-153 and 199-202 in the reference
 * example): key_nope_2d is [kv_rows, 512] bf16 and is used as it is,
 * k_nope_scales is not read (may be NULL).  Everything else as above; the
 * workspace is the one pto_sfa_quant_workspace_bytes reports.
 */
int pto_sfa_bf16kv_launch(const PtoSfaQuantArgs *args, void *hip_stream);

/*
 * The same attention over the packed cache of sparse_attention_antiquant_d
 * (sparse_attention_antiquant_impl.py:45-85 in the reference example; packing
 * deepseekv32_sparse_attention_antiquant.py:258-268):
 *
 *   nope_cache [kv_rows, 656] int8: bytes 0..511 the int8 latent values,
 *                                   512..639 the 64 bf16 rope values,
 *                                   640..655 the 4 fp32 scales
 *
 * All other tensors, the arithmetic, cur_seq, clamping, constraints, workspace
 * and num_splits are those of PtoSfaQuantArgs.
 */
typedef struct PtoSaAntiquantArgs {
    const void *query_nope;
    const void *query_rope;
    const void *nope_cache;
    const int32_t *topk_indices;
    const int32_t *block_table;
    const int32_t *kv_act_seqs;
    void *attention_out;
    void *workspace;
    size_t workspace_bytes;
    int64_t b;
    int64_t s1;
    int64_t nq;
    int64_t n_kv;
    int64_t topk;
    int64_t block_size;
    int64_t max_blocknum_perbatch;
    int64_t kv_rows;
    float softmax_scale;
    int32_t num_splits;
} PtoSaAntiquantArgs;

int pto_sa_antiquant_workspace_bytes(const PtoSaAntiquantArgs *args, size_t *bytes);
int pto_sa_antiquant_launch(const PtoSaAntiquantArgs *args, void *hip_stream);

/*
 * Lightning indexer, decode form (lightning_indexer_quant_impl.py:52-82 in the
 * reference example):
 *
 *   idx_query       [t, n_heads, head_dim]                 int8   t = b*s1
 *   idx_query_scale [t, n_heads]                           q_scale_dtype
 *   idx_key_cache   [block_num, block_size, 1, head_dim]   int8
 *   idx_key_scale   [block_num, block_size, 1]             k_scale_dtype
 *   idx_weight      [t, n_heads]                           weight_dtype
 *   act_seq_key     [b]                                    int32
 *   block_table     [b, max_blocknum_perbatch]             int32
 *   topk_res        [t, 1, selected_count]                 int32  written in place
 *
 * score[s, j] = (sum_h w_scale[s,h] * fp16(relu(q[s,h,:] . k[j,:]) / 2048)) * k_scale[j]
 * with the head sum taken in fp32, h ascending, product rounded before the add;
 * w_scale = fp16(q_scale * weight) when both are fp16, else the fp32 product.
 * Query token s of batch bi sees positions 0 .. act_seq_key[bi] - (s1-1-s) - 1;
 * the selected_count best are written ordered by (score descending, position
 * ascending), padded with -1.
 *
 * Constraints: n_heads == 64, head_dim == 128, 1 <= selected_count <= 2048,
 * max_blocknum_perbatch * block_size <= 131072, block_size a multiple of 32,
 * t <= 65535.  Alignment: idx_query, idx_key_cache and workspace 16 bytes, the
 * int32 tensors 4 bytes, scales and weights their element size.
 */
typedef struct PtoLiDecodeArgs {
    const int8_t *idx_query;
    const void *idx_query_scale;
    const int8_t *idx_key_cache;
    const void *idx_key_scale;
    const void *idx_weight;
    const int32_t *act_seq_key;
    const int32_t *block_table;
    int32_t *topk_res;
    void *workspace;
    size_t workspace_bytes;
    int64_t t;
    int64_t b;
    int64_t n_heads;
    int64_t head_dim;
    int64_t block_num;
    int64_t block_size;
    int64_t max_blocknum_perbatch;
    int64_t selected_count;
    int32_t q_scale_dtype;
    int32_t k_scale_dtype;
    int32_t weight_dtype;
    int32_t arith_variant;   /* 0: the arithmetic above.  1: that of the reference's chained C++ operator
                                (framework/src/operator/models/deepseek_v3.2_exp/lightning_indexer.cpp:149-197):
                                v = fp16(q.k / 2048); v = fp16(fp16(v * q_scale) * k_scale); v = max(v, 0);
                                v = fp16(v * weight); score = fp32 sum over heads, h ascending.  All three
                                dtype codes must be PTO_DT_FP16. */
} PtoLiDecodeArgs;

int pto_li_decode_workspace_bytes(const PtoLiDecodeArgs *args, size_t *bytes);
int pto_li_decode_launch(const PtoLiDecodeArgs *args, void *hip_stream);

/*
 * Lightning-indexer prolog, quantized (lightning_indexer_prolog_quant_impl.py:325-504
 * in the reference example; torch golden
 * deepseekv32_lightning_indexer_prolog_quant.py:216-281):
 *
 *   x              [t, h]                        bf16
 *   q_norm         [t, q_lora_rank]              int8
 *   q_norm_scale   [t, 1]                        fp32
 *   w_qb           [q_lora_rank, n_heads*128]    int8   row-major (the reference passes
 *                                                       its NPU fractal form of this matrix)
 *   w_qb_scale     [n_heads*128, 1]              fp32
 *   wk             [h, 128]                      bf16   row-major
 *   w_proj         [h, n_heads]                  bf16   row-major
 *   ln_gamma_k, ln_beta_k  [128]                 bf16
 *   cos_idx_rope, sin_idx_rope  [t, 64]          bf16
 *   hadamard_q, hadamard_k      [128, 128]       bf16
 *   k_cache        [block_num, block_size, 1, 128]  int8   rows k_cache_index[i] rewritten
 *   k_cache_scale  [block_num, block_size, 1, 1]    fp16   same rows
 *   k_cache_index  [t]                           int64  physical cache row of each token
 *   q_int8         [t, n_heads, 128]             int8   written
 *   q_scale        [t, n_heads, 1]               fp16   written
 *   weights        [t, n_heads]                  fp16   written
 *
 * Every fp32 sum has a fixed order, so results are reproducible bit for bit:
 * sums over h in blocks of 64 (ascending inside a block), eight consecutive block
 * sums added ascending into a group sum and the group sums added ascending; the
 * 128-term Hadamard sums ascending; the layer-norm means as balanced trees over
 * neighbouring channels.  A row whose values are all zero quantises to zeros with
 * scale 0.  Cache indices outside [0, cache_rows) are skipped.
 *
 * Constraints: head_dim 128, rope 64, 1 <= n_heads <= 64, q_lora_rank in
 * {512, 1024, 1536}, h a positive multiple of 64 up to 12288, t >= 1.
 */
typedef struct PtoLiPrologQuantArgs {
    const void *x;
    const int8_t *q_norm;
    const float *q_norm_scale;
    const int8_t *w_qb;
    const float *w_qb_scale;
    const void *wk;
    const void *w_proj;
    const void *ln_gamma_k;
    const void *ln_beta_k;
    const void *cos_idx_rope;
    const void *sin_idx_rope;
    const void *hadamard_q;
    const void *hadamard_k;
    int8_t *k_cache;
    void *k_cache_scale;
    const int64_t *k_cache_index;
    int8_t *q_int8;
    void *q_scale;
    void *weights;
    void *workspace;
    size_t workspace_bytes;
    int64_t t;
    int64_t h;
    int64_t q_lora_rank;
    int64_t n_heads;
    int64_t cache_rows;   /* block_num * block_size */
    float eps;            /* layer-norm epsilon (attrs.eps) */
    int32_t sum_mode;     /* how the fp32 sums are taken from 64 tokens on (below that always in the fixed order
                             above, bit-reproducible):
                             0 (what a zero-initialised struct gives): the query rows' Hadamard sums on the matrix
                               cores -- the same exact bf16 products added in the cores' order, so q_int8 may
                               differ by one step and q_scale in its last bit in rare rows, which the reference's
                               acceptance rule for these two outputs allows
                               (deepseekv32_lightning_indexer_prolog_quant.py:424-425); the key row and the
                               weights, for which that rule allows no outlier (:426-428), keep the fixed order;
                             1: every sum in its fixed order;
                             2: as 0, and the sums over h on the matrix cores as well (n_heads a multiple of 8): the
                               fastest form; the key row's scale and the weights may then differ by one rounding
                               step of their bf16 intermediate in rare entries. */
} PtoLiPrologQuantArgs;

int pto_li_prolog_quant_workspace_bytes(const PtoLiPrologQuantArgs *args, size_t *bytes);
int pto_li_prolog_quant_launch(const PtoLiPrologQuantArgs *args, void *hip_stream);

/*
 * MLA prolog, quantized (mla_prolog_quant_impl.py:502-707 in the reference example;
 * torch golden deepseekv32_mla_prolog_quant.py:137-282), in the variant of the
 * reference's enabled case: bf16 down-projections, int8 w_uq_qr with per-column
 * scales, int8 latent cache with four fp32 scales per token, cache mode PA_BSND.
 *
 *   token_x        [t, h]                        bf16
 *   w_dq           [h, q_lora_rank]              bf16   row-major
 *   w_uq_qr        [q_lora_rank, n_heads*192]    int8   row-major; per head 128 nope + 64 rope columns
 *   dequant_scale  [n_heads*192, 1]              fp32
 *   w_uk           [n_heads, 128, 512]           bf16
 *   w_dkv_kr       [h, 576]                      bf16   row-major; 512 latent + 64 rope columns
 *   gamma_cq [q_lora_rank], gamma_ckv [512]      bf16
 *   cos, sin       [t, 64]                       bf16
 *   cache_index    [t]                           int64  physical cache row of each token
 *   kv_cache       [block_num, block_size, 1, 512]  int8   rows cache_index[i] rewritten
 *   kr_cache       [block_num, block_size, 1, 64]   bf16   same rows
 *   k_scale_cache  [block_num, block_size, 1, 4]    fp32   same rows
 *   q_norm_out         [t, q_lora_rank]          int8   written
 *   q_norm_scale_out   [t, 1]                    fp32   written
 *   query_nope_out     [t, n_heads, 512]         bf16   written
 *   query_rope_out     [t, n_heads, 64]          bf16   written
 *
 * Every fp32 sum has a fixed order (hidden-axis sums as in the indexer prolog; RMS
 * sums as a balanced tree over each slab of 128 channels, slabs ascending; the
 * 128-term sums against w_uk ascending), so results are reproducible bit for bit.
 * RMS norm: v / sqrt(mean(v^2) + epsilon) * gamma (epsilon 0 = the torch golden).
 *
 * Constraints: q_lora_rank in {512, 1024, 1536}, h a positive multiple of 64 up to
 * 16384, n_heads even, t >= 1.
 */
typedef struct PtoMlaPrologQuantArgs {
    const void *token_x;
    const void *w_dq;
    const int8_t *w_uq_qr;
    const float *dequant_scale;
    const void *w_uk;
    const void *w_dkv_kr;
    const void *gamma_cq;
    const void *gamma_ckv;
    const void *cos;
    const void *sin;
    const int64_t *cache_index;
    int8_t *kv_cache;
    void *kr_cache;
    float *k_scale_cache;
    int8_t *q_norm_out;
    float *q_norm_scale_out;
    void *query_nope_out;
    void *query_rope_out;
    void *workspace;
    size_t workspace_bytes;
    int64_t t;
    int64_t h;
    int64_t q_lora_rank;
    int64_t n_heads;
    int64_t cache_rows;   /* block_num * block_size */
    float epsilon_cq;
    float epsilon_ckv;
    int32_t absorb_exact; /* query_nope = (query . w_uk): 1 = fixed-order fp32 sums (bit-reproducible, the statement
                             above); 0 = on the matrix cores: the same exact bf16 products summed in fp32 in the
                             cores' order, so some results differ in the last bf16 bit -- inside the reference's
                             own acceptance rule for this output (deepseekv32_mla_prolog_quant.py:668-692), which
                             only feeds the attention.  With at most 8 tokens every other output is the same either
                             way; from 9 tokens on, 0 also takes the sums over the hidden axis on the matrix cores
                             (int8 latents then differ by one step in rare entries, inside the same rule) and 1
                             keeps every sum in its fixed order. */
    int32_t reserved;
} PtoMlaPrologQuantArgs;

int pto_mla_prolog_quant_workspace_bytes(const PtoMlaPrologQuantArgs *args, size_t *bytes);
int pto_mla_prolog_quant_launch(const PtoMlaPrologQuantArgs *args, void *hip_stream);

/*
 * MLA prolog + lightning-indexer prolog as one operator (mla_indexer_prolog_quant_d/_p,
 * examples/models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:49-138, 141-256 in the
 * reference): the MLA prolog runs first; its int8 normalised query latent and that latent's
 * scale -- intermediates the reference's caller never sees (:218-219) -- feed the indexer
 * prolog; hidden states, rope tables and cache index are shared.
 *
 *   mla      as for pto_mla_prolog_quant_launch.  q_norm_out / q_norm_scale_out may be NULL:
 *            the two intermediates then live in the common workspace.  workspace and
 *            workspace_bytes of this part are ignored.
 *   indexer  as for pto_li_prolog_quant_launch, of which x, q_norm, q_norm_scale,
 *            cos_idx_rope, sin_idx_rope, k_cache_index, t, h, q_lora_rank, workspace and
 *            workspace_bytes are ignored: taken from the MLA part and the common workspace.
 *   workspace  pto_mla_indexer_prolog_quant_workspace_bytes() bytes, 256-byte aligned: the
 *            intermediates, then the partial sums of the MLA half, then those of the indexer half.
 * Five kernels on the given stream, nothing else (the last launches of the two halves do not
 * depend on each other and run as one); errors as for the two operators.
 */
typedef struct PtoMlaIndexerPrologQuantArgs {
    PtoMlaPrologQuantArgs mla;
    PtoLiPrologQuantArgs indexer;
    void *workspace;
    size_t workspace_bytes;
} PtoMlaIndexerPrologQuantArgs;

int pto_mla_indexer_prolog_quant_workspace_bytes(const PtoMlaIndexerPrologQuantArgs *args, size_t *bytes);
int pto_mla_indexer_prolog_quant_launch(const PtoMlaIndexerPrologQuantArgs *args, void *hip_stream);

/* Thread-local description of the last error on this thread ("" if none). */
const char *pto_last_error(void);

/* Library version, "major.minor.patch". */
const char *pto_version(void);

/*
 * Revision of the argument structs above.  The structs carry no size field and have grown between revisions
 * (revision 2 added absorb_exact and a reserved word to PtoMlaPrologQuantArgs, revision 1 was library 0.1.0): a
 * caller built against another revision would hand over structs of another size.  Compare once after loading:
 * pto_abi_revision() == PTO_ABI_REVISION, else do not call the launch functions of this library.
 */
#define PTO_ABI_REVISION 2
int pto_abi_revision(void);

#ifdef __cplusplus
}
#endif
#endif /* PYPTO_AMD_SFA_H */
