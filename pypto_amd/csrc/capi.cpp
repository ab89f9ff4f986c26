// C ABI of the library: argument validation, workspace sizing, launch heuristics.
// Declarations and the reference interfaces they stand in for: include/pypto_amd_sfa.h.
#include "pypto_amd_sfa.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "li_kernels.h"
#include "lip_kernels.h"
#include "prolog_fused.h"
#include "mlap_kernels.h"
#include "sfa_kernels.h"

// Scratch memory of pto_sfa_quant_launch_static: the partial results of the key splits live here
// instead of in a caller workspace.  One copy per GPU the library's code object is loaded on, held
// until the process ends.  In host code the name below is only a handle; the device address is asked
// for once per device (scratch_of) and that pointer is what the kernels get.
constexpr size_t SFA_STATIC_SCRATCH_BYTES = (size_t)40 << 20;
static __device__ __align__(256) unsigned char scratch[SFA_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace

namespace pto {
// compute units of the current device (one query per device ordinal, then cached)
int cu_count()
{
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> cached[MAX_DEVICES];
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (dev >= 0 && dev < MAX_DEVICES) {
        n = cached[dev].load(std::memory_order_relaxed);
        if (n > 0) return n;
    }
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    if (dev >= 0 && dev < MAX_DEVICES) cached[dev].store(n, std::memory_order_relaxed);
    return n;
}
}  // namespace pto

namespace {

using pto::cu_count;

// device address of this device's copy of the scratch array (NULL and *err set on failure)
void *scratch_of(int dev, hipError_t *err)
{
    constexpr int MAX_DEVICES = 64;
    static std::atomic<void *> ptrs[MAX_DEVICES];
    static std::mutex mu;
    *err = hipSuccess;
    if (dev < 0 || dev >= MAX_DEVICES) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    void *p = ptrs[dev].load(std::memory_order_acquire);
    if (p) return p;
    std::lock_guard<std::mutex> lock(mu);
    p = ptrs[dev].load(std::memory_order_relaxed);
    if (p) return p;
    void *addr = nullptr;
    *err = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));     // the current device is dev (checked by the caller)
    if (*err != hipSuccess || !addr) {
        if (*err == hipSuccess) *err = hipErrorInvalidSymbol;
        return nullptr;
    }
    ptrs[dev].store(addr, std::memory_order_release);
    return addr;
}

struct SfaPlan {
    int waves;
    int hgroups;
    int nsplit;
    int whole_slots;      // rows 0 .. 8 * whole_slots - 1 are not split
    size_t part_o_bytes;
    size_t part_ml_bytes;
    size_t predeq_bytes;  // the whole cache de-quantised once, behind the partial results (0: not worth it)
    size_t predeq_offset; // where in the workspace
};

constexpr size_t SFA_PREDEQ_MAX_BYTES = (size_t)64 << 20;

int sfa_check(const PtoSfaQuantArgs *a)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "sfa: args is NULL");
    if (a->b < 1 || a->s1 < 1 || a->nq < 1) return fail(PTO_E_INVALID_ARG, "sfa: b, s1, nq must be >= 1");
    if (a->n_kv != 1) return fail(PTO_E_INVALID_ARG, "sfa: n_kv must be 1 (got %lld)", (long long)a->n_kv);
    if (a->topk < 1) return fail(PTO_E_INVALID_ARG, "sfa: topk must be >= 1");
    if (a->block_size < 1 || a->max_blocknum_perbatch < 1)
        return fail(PTO_E_INVALID_ARG, "sfa: block_size and max_blocknum_perbatch must be >= 1");
    if (a->kv_rows < 1) return fail(PTO_E_INVALID_ARG, "sfa: kv_rows must be >= 1");
    if (a->b > (1ll << 24) || a->s1 > (1ll << 24) || a->b * a->s1 > (1ll << 24) || a->nq > 65536 || a->topk > (1ll << 24) ||
        a->kv_rows > 0x7fffffffll || a->block_size > (1ll << 30) || a->max_blocknum_perbatch > (1ll << 30))
        return fail(PTO_E_INVALID_ARG, "sfa: shape out of the supported range");
    if (a->num_splits < 0) return fail(PTO_E_INVALID_ARG, "sfa: num_splits must be >= 0");
    if (!std::isfinite(a->softmax_scale)) return fail(PTO_E_INVALID_ARG, "sfa: softmax_scale is not finite");
    return PTO_OK;
}

// max_bytes: most bytes of partial results the caller can hold; the automatic choice (num_splits = 0) then takes the
// best split count among those that fit (an explicit count is the caller's own business)
SfaPlan sfa_plan(const PtoSfaQuantArgs *a, const size_t max_bytes = ~(size_t)0)
{
    SfaPlan pl;
    pl.waves = a->nq > 64 ? 4 : (a->nq > 32 ? 2 : 1);
    const int heads_per_wg = 32 * pl.waves;
    pl.hgroups = (int)((a->nq + heads_per_wg - 1) / heads_per_wg);
    const long long rows = a->b * a->s1;
    const int tiles = (int)((a->topk + pto::SFA_KEY_TILE - 1) / pto::SFA_KEY_TILE);
    const int min_split = (int)((a->topk + pto::SFA_MAX_CHUNK - 1) / pto::SFA_MAX_CHUNK);
    int ns = a->num_splits;
    if (ns == 0) {
        // The split count with the shortest schedule.  The workgroups of a row share an XCD (row t on XCD t % 8,
        // for the row's queries in that XCD's L2) and a compute unit holds one workgroup, so the fullest XCD runs
        // ceil(its workgroups / its CUs) rounds, each as long as a split's tiles plus the fixed cost of a workgroup
        // (query staging, row table, first tile, writing the partial results: about five and a half tiles' time;
        // three when nothing is split); the merge launch costs about a tile plus a tile per hundred partial rows.
        // Filling every XCD exactly once wins where the batch allows it; a batch that does not divide the CUs
        // gets fewer, longer splits rather than a second round that is nearly empty, and a batch of more rows
        // than CUs is split where shorter workgroups fill its last round better (300 rows: three rounds of half
        // rows instead of two of whole ones).  A split shorter than four tiles is all prologue.
        // (a size query on a host without a device plans for the 256 CUs of an MI355X; a launch there fails)
        const int cus = cu_count() > 0 ? cu_count() : 256;
        const long long xcd_cus = cus / 8 > 0 ? cus / 8 : 1;
        const long long xcd_rows = (rows + 7) / 8;
        const int max_split = tiles / 4 > 0 ? tiles / 4 : 1;
        double best = -1.0;
        if (cus % 8 != 0) {
            // not the layout the schedule model describes (a partitioned device, another part): one workgroup per
            // compute unit, as many splits as that takes
            const long long per_split = rows * pl.hgroups;
            ns = (int)((cus + per_split - 1) / per_split);
            ns = ns > max_split ? max_split : ns;
            while (ns > 1 && ns > min_split && (size_t)rows * ns * a->nq * (512 * sizeof(uint16_t) + 2 * sizeof(float)) > max_bytes) --ns;
        }
        for (int s = 1; s <= max_split && cus % 8 == 0; ++s) {
            if (s > 1 && s >= min_split && (size_t)rows * s * a->nq * (512 * sizeof(uint16_t) + 2 * sizeof(float)) > max_bytes) break;
            const long long rounds = (xcd_rows * pl.hgroups * s + xcd_cus - 1) / xcd_cus;
            const double merge = s == 1 ? 0.0 : 1.0 + 0.01 * (double)rows * s * pl.hgroups;
            const double cost = (double)rounds * ((tiles + s - 1) / s + (s == 1 ? 3.0 : 5.5)) + merge;
            if (best < 0.0 || cost < best) {
                best = cost;
                ns = s;
            }
        }
    }
    ns = ns < min_split ? min_split : ns;
    ns = ns > tiles ? tiles : ns;
    ns = ns < 1 ? 1 : ns;
    pl.nsplit = ns;
    pl.whole_slots = 0;
    long long split_rows = rows;
    if (a->num_splits == 0 && min_split == 1) {
        // More rows than compute units: the full rounds of whole rows first, then the rows left over dealt out in
        // as many pieces as fill one more round (300 rows on 256 CUs: 32 whole rows per XCD, the other five or
        // six in five pieces each), where that beats the best uniform split above.
        const int cus = cu_count() > 0 ? cu_count() : 256;
        const long long xcd_cus = cus / 8 > 0 ? cus / 8 : 1;
        const long long xcd_rows = (rows + 7) / 8;
        const long long per_round = cus % 8 == 0 ? xcd_cus / pl.hgroups : 0;   // rows of an XCD that one round holds
        const long long full = per_round > 0 ? xcd_rows / per_round : 0;
        const long long rem = per_round > 0 ? xcd_rows - full * per_round : 0;
        if (full >= 1 && rem >= 1) {
            int sb = (int)(per_round / rem);
            const int max_split = tiles / 4 > 0 ? tiles / 4 : 1;
            sb = sb > max_split ? max_split : sb;
            const long long rows_b = rows - 8 * full * per_round;         // rows 8 * whole_slots and up
            if (sb >= 2 && rows_b > 0 &&
                (size_t)rows_b * sb * a->nq * (512 * sizeof(uint16_t) + 2 * sizeof(float)) <= max_bytes) {
                const double merge = 1.0 + 0.01 * (double)rows_b * sb * pl.hgroups;
                const double cost = (double)full * (tiles + 3.0) + ((tiles + sb - 1) / sb + 5.5) + merge;
                const long long rounds_u = (xcd_rows * pl.hgroups * ns + xcd_cus - 1) / xcd_cus;
                const double cost_u = (double)rounds_u * ((tiles + ns - 1) / ns + (ns == 1 ? 3.0 : 5.5)) +
                                      (ns == 1 ? 0.0 : 1.0 + 0.01 * (double)rows * ns * pl.hgroups);
                if (cost < cost_u) {
                    pl.nsplit = sb;
                    pl.whole_slots = (int)(full * per_round);
                    split_rows = rows_b;
                }
            }
        }
    }
    if (pl.nsplit > 1) {
        pl.part_o_bytes = (size_t)split_rows * pl.nsplit * a->nq * 512 * sizeof(uint16_t);
        pl.part_ml_bytes = (size_t)split_rows * pl.nsplit * a->nq * 2 * sizeof(float);
    } else {
        pl.part_o_bytes = pl.part_ml_bytes = 0;
    }
    // A launch that selects every cache row many times over (a prefill chunk: thousands of query rows over a few
    // thousand keys) de-quantises the cache once into the workspace and attends over the bf16 rows -- the same
    // bits, since the kernel's bf16-cache form reads exactly what its int8 form converts to, without the per-tile
    // conversion (8 % at 4096 query rows over 4096 keys).  Only for caches that fit a modest workspace.
    pl.predeq_offset = (pl.part_o_bytes + pl.part_ml_bytes + 255) / 256 * 256;
    pl.predeq_bytes = 0;
    const size_t dq = (size_t)a->kv_rows * 512 * sizeof(uint16_t);
    if (rows * a->topk >= 8 * a->kv_rows && dq <= SFA_PREDEQ_MAX_BYTES && pl.predeq_offset + dq <= max_bytes) pl.predeq_bytes = dq;
    return pl;
}

size_t sfa_ws_bytes(const SfaPlan &pl) { return pl.predeq_bytes ? pl.predeq_offset + pl.predeq_bytes : pl.part_o_bytes + pl.part_ml_bytes; }

constexpr int PACKED_ROW_BYTES = 656;     // 512 int8 | 64 bf16 | 4 fp32

// the packed-cache arguments seen as the three-array ones (the cache pointers are filled in by the caller)
PtoSfaQuantArgs unpacked_view(const PtoSaAntiquantArgs *a)
{
    PtoSfaQuantArgs q;
    std::memset(&q, 0, sizeof(q));
    q.query_nope = a->query_nope;
    q.query_rope = a->query_rope;
    q.key_nope_2d = a->nope_cache;
    q.key_rope_2d = a->nope_cache;
    q.k_nope_scales = a->nope_cache;
    q.topk_indices = a->topk_indices;
    q.block_table = a->block_table;
    q.kv_act_seqs = a->kv_act_seqs;
    q.attention_out = a->attention_out;
    q.workspace = a->workspace;
    q.workspace_bytes = a->workspace_bytes;
    q.b = a->b;
    q.s1 = a->s1;
    q.nq = a->nq;
    q.n_kv = a->n_kv;
    q.topk = a->topk;
    q.block_size = a->block_size;
    q.max_blocknum_perbatch = a->max_blocknum_perbatch;
    q.kv_rows = a->kv_rows;
    q.softmax_scale = a->softmax_scale;
    q.num_splits = a->num_splits;
    return q;
}

// checked arguments -> kernel parameters -> launch; the cache is given as three (base, row pitch) pairs
int sfa_enqueue(const PtoSfaQuantArgs *a, const int8_t *kn, int kn_pitch, const uint8_t *kr, int kr_pitch, const uint8_t *ksc,
                int ksc_pitch, void *hip_stream, bool kn_bf16 = false, const size_t plan_limit = ~(size_t)0)
{
    if (cu_count() <= 0) return fail(PTO_E_NO_DEVICE, "sfa: no usable device is current");
    const SfaPlan pl = sfa_plan(a, plan_limit);
    if (((long long)(a->b * a->s1) + 7) / 8 * 8 * pl.hgroups * pl.nsplit > 0x7fffffffll)     // (an upper bound of the grid)
        return fail(PTO_E_INVALID_ARG, "sfa: rows x head groups x key splits exceeds the largest launch");
    {
        const void *al16[] = {a->query_nope, a->query_rope, kn, kr, ksc, a->attention_out, a->workspace};
        for (const void *ptr : al16)
            if (reinterpret_cast<uintptr_t>(ptr) & 15)
                return fail(PTO_E_INVALID_ARG, "sfa: query, cache, output and workspace pointers must be 16-byte aligned");
        const void *al4[] = {a->topk_indices, a->block_table, a->kv_act_seqs};
        for (const void *ptr : al4)
            if (reinterpret_cast<uintptr_t>(ptr) & 3)
                return fail(PTO_E_INVALID_ARG, "sfa: index, block-table and length pointers must be 4-byte aligned");
    }
    const bool predeq = pl.predeq_bytes != 0 && !kn_bf16;
    const size_t need = predeq ? sfa_ws_bytes(pl) : pl.part_o_bytes + pl.part_ml_bytes;
    if (need > 0 && (!a->workspace || a->workspace_bytes < need))
        return fail(PTO_E_WORKSPACE, "sfa: workspace of %zu bytes required, %zu given", need, a->workspace ? a->workspace_bytes : (size_t)0);
    if (predeq) {
        uint16_t *dq = reinterpret_cast<uint16_t *>(static_cast<char *>(a->workspace) + pl.predeq_offset);
        hipError_t e = pto::sfa_dequant_cache(kn, kn_pitch, ksc, ksc_pitch, dq, a->kv_rows, static_cast<hipStream_t>(hip_stream));
        if (e != hipSuccess) return fail(PTO_E_LAUNCH, "sfa: launch failed: %s", hipGetErrorString(e));
        kn = reinterpret_cast<const int8_t *>(dq);
        kn_pitch = 1024;
        kn_bf16 = true;
    }

    pto::SfaParams p;
    p.q_nope = static_cast<const uint16_t *>(a->query_nope);
    p.q_rope = static_cast<const uint16_t *>(a->query_rope);
    p.kn = kn;
    p.kr = kr;
    p.ksc = ksc;
    p.kn_pitch = kn_pitch;
    p.kr_pitch = kr_pitch;
    p.ksc_pitch = ksc_pitch;
    p.kn_bf16 = kn_bf16 ? 1 : 0;
    p.topk_idx = a->topk_indices;
    p.bt = a->block_table;
    p.act = a->kv_act_seqs;
    p.out = static_cast<uint16_t *>(a->attention_out);
    p.part_o = static_cast<uint16_t *>(a->workspace);
    p.part_ml = pl.part_ml_bytes > 0 ? reinterpret_cast<float *>(static_cast<char *>(a->workspace) + pl.part_o_bytes) : nullptr;
    p.kv_rows = a->kv_rows;
    p.T = (int)(a->b * a->s1);
    p.S1 = (int)a->s1;
    p.NQ = (int)a->nq;
    p.topk = (int)a->topk;
    p.bs = (int)a->block_size;
    p.maxblk = (int)a->max_blocknum_perbatch;
    p.nsplit = pl.nsplit;
    p.whole_slots = pl.whole_slots;
    p.hgroups = pl.hgroups;
    p.waves = pl.waves;
    p.scale_log2 = a->softmax_scale * 1.4426950408889634f;
    hipError_t e = pto::sfa_launch(p, static_cast<hipStream_t>(hip_stream));
    if (e == hipErrorNoBinaryForGpu || e == hipErrorInvalidDeviceFunction)
        return fail(PTO_E_NO_DEVICE, "sfa: the library holds gfx950 code only: %s", hipGetErrorString(e));
    if (e != hipSuccess) return fail(PTO_E_LAUNCH, "sfa: launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

constexpr long long LI_MAX_SEQ_HOST = pto::LI_MAX_SEQ;

int li_check(const PtoLiDecodeArgs *a)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "li: args is NULL");
    if (a->t < 1 || a->b < 1 || a->t % a->b != 0) return fail(PTO_E_INVALID_ARG, "li: t must be a positive multiple of b");
    if (a->n_heads != 64 || a->head_dim != 128)
        return fail(PTO_E_INVALID_ARG, "li: n_heads must be 64 and head_dim 128 (got %lld, %lld)", (long long)a->n_heads,
                    (long long)a->head_dim);
    if (a->selected_count < 1 || a->selected_count > pto::LI_MAX_SELECT)
        return fail(PTO_E_INVALID_ARG, "li: selected_count must be in [1, %d]", pto::LI_MAX_SELECT);
    if (a->block_size < 32 || a->block_size % 32 != 0) return fail(PTO_E_INVALID_ARG, "li: block_size must be a multiple of 32");
    if (a->block_num < 1 || a->max_blocknum_perbatch < 1) return fail(PTO_E_INVALID_ARG, "li: block_num and max_blocknum_perbatch must be >= 1");
    if (a->max_blocknum_perbatch * a->block_size > pto::LI_MAX_SEQ)
        return fail(PTO_E_INVALID_ARG, "li: max_blocknum_perbatch * block_size exceeds %d", pto::LI_MAX_SEQ);
    if (a->t > (1ll << 20) || a->block_num > 0x7fffffffll || a->block_size > LI_MAX_SEQ_HOST || a->block_num * a->block_size > 0x7fffffffll)
        return fail(PTO_E_INVALID_ARG, "li: shape out of the supported range");
    if (a->t > pto::LI_MAX_BALANCED_TOKENS && a->t > 65535)
        return fail(PTO_E_INVALID_ARG, "li: at most 65535 query tokens per launch (got %lld)", (long long)a->t);
    if (a->arith_variant != 0 && a->arith_variant != 1) return fail(PTO_E_INVALID_ARG, "li: arith_variant must be 0 or 1");
    if (a->arith_variant == 1 &&
        (a->q_scale_dtype != PTO_DT_FP16 || a->k_scale_dtype != PTO_DT_FP16 || a->weight_dtype != PTO_DT_FP16))
        return fail(PTO_E_INVALID_ARG, "li: arith_variant 1 takes fp16 scales and weights");
    const int dts[3] = {a->q_scale_dtype, a->k_scale_dtype, a->weight_dtype};
    for (int d : dts)
        if (d != PTO_DT_FP16 && d != PTO_DT_FP32 && d != PTO_DT_BF16) return fail(PTO_E_INVALID_ARG, "li: unknown dtype code %d", d);
    return PTO_OK;
}

size_t li_ws_bytes(const PtoLiDecodeArgs *a)
{
    // score rows [t, max_blocknum_perbatch*block_size] fp32, then one sampled score per 16 positions
    const size_t stride = (size_t)a->max_blocknum_perbatch * a->block_size;
    return (size_t)a->t * (stride + stride / pto::LI_SAMPLE_GROUP) * sizeof(float);
}

int lip_check(const PtoLiPrologQuantArgs *a)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "li_prolog: args is NULL");
    if (a->t < 1 || a->t > (1ll << 20)) return fail(PTO_E_INVALID_ARG, "li_prolog: t must be in [1, 2^20]");
    if (a->n_heads < 1 || a->n_heads > pto::LIP_MAX_HEADS)
        return fail(PTO_E_INVALID_ARG, "li_prolog: n_heads must be in [1, %d] (got %lld)", pto::LIP_MAX_HEADS, (long long)a->n_heads);
    static_assert(pto::LIP_MAX_QLORA == 1536, "the list below follows the kernel's instantiations");
    if (a->q_lora_rank != 512 && a->q_lora_rank != 1024 && a->q_lora_rank != 1536)
        return fail(PTO_E_INVALID_ARG, "li_prolog: q_lora_rank must be 512, 1024 or 1536 (got %lld)", (long long)a->q_lora_rank);
    const long long max_h = (long long)pto::LIP_MAX_XGROUPS * pto::LIP_XGROUP * pto::LIP_XBLOCK;
    if (a->h < pto::LIP_XBLOCK || a->h % pto::LIP_XBLOCK != 0 || a->h > max_h)
        return fail(PTO_E_INVALID_ARG, "li_prolog: h must be a positive multiple of %d, at most %lld (got %lld)", pto::LIP_XBLOCK,
                    max_h, (long long)a->h);
    if (a->cache_rows < 1 || a->cache_rows > 0x7fffffffll) return fail(PTO_E_INVALID_ARG, "li_prolog: cache_rows out of range");
    if (!std::isfinite(a->eps) || a->eps < 0) return fail(PTO_E_INVALID_ARG, "li_prolog: eps must be finite and >= 0");
    return PTO_OK;
}

// [4 partial int32 projections | block sums over the hidden axis]
size_t lip_qpart_bytes(const PtoLiPrologQuantArgs *a)
{
    return (size_t)pto::LIP_KSPLIT * a->t * a->n_heads * pto::LIP_DIM * sizeof(int32_t);
}
size_t lip_ws_bytes(const PtoLiPrologQuantArgs *a)
{
    return lip_qpart_bytes(a) + (size_t)(a->h / pto::LIP_XBLOCK) * a->t * pto::LIP_XCOLS * sizeof(float);
}

int mlap_check(const PtoMlaPrologQuantArgs *a)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "mla_prolog: args is NULL");
    if (a->t < 1 || a->t > (1ll << 20)) return fail(PTO_E_INVALID_ARG, "mla_prolog: t must be in [1, 2^20]");
    if (a->n_heads < 2 || a->n_heads % 2 != 0 || a->n_heads > 1024)
        return fail(PTO_E_INVALID_ARG, "mla_prolog: n_heads must be even, in [2, 1024] (got %lld)", (long long)a->n_heads);
    if (a->q_lora_rank != 512 && a->q_lora_rank != 1024 && a->q_lora_rank != 1536)
        return fail(PTO_E_INVALID_ARG, "mla_prolog: q_lora_rank must be 512, 1024 or 1536 (got %lld)", (long long)a->q_lora_rank);
    const long long max_h = (long long)pto::MLAP_MAX_XGROUPS * pto::MLAP_XGROUP * pto::MLAP_XBLOCK;
    if (a->h < pto::MLAP_XBLOCK || a->h % pto::MLAP_XBLOCK != 0 || a->h > max_h)
        return fail(PTO_E_INVALID_ARG, "mla_prolog: h must be a positive multiple of %d, at most %lld (got %lld)", pto::MLAP_XBLOCK,
                    max_h, (long long)a->h);
    if (a->cache_rows < 1 || a->cache_rows > 0x7fffffffll) return fail(PTO_E_INVALID_ARG, "mla_prolog: cache_rows out of range");
    if (!std::isfinite(a->epsilon_cq) || a->epsilon_cq < 0 || !std::isfinite(a->epsilon_ckv) || a->epsilon_ckv < 0)
        return fail(PTO_E_INVALID_ARG, "mla_prolog: epsilons must be finite and >= 0");
    return PTO_OK;
}

// [group sums over the hidden axis | 4 partial int32 projections]
size_t mlap_xpart_bytes(const PtoMlaPrologQuantArgs *a)
{
    const size_t rows = (size_t)pto::mlap_xpart_rows((int)a->h, (int)a->t);
    const size_t bytes = rows * a->t * (a->q_lora_rank + pto::MLAP_KV + pto::MLAP_ROPE) * sizeof(float);
    return (bytes + 255) & ~(size_t)255;
}
size_t mlap_ws_bytes(const PtoMlaPrologQuantArgs *a)
{
    return mlap_xpart_bytes(a) + (size_t)pto::QPROJ_KSPLIT_HOST * a->t * a->n_heads * pto::MLAP_QHEAD * sizeof(int32_t);
}

}  // namespace

extern "C" {

const char *pto_last_error(void) { return g_err; }

const char *pto_version(void) { return "0.6.0"; }

int pto_abi_revision(void) { return PTO_ABI_REVISION; }

int pto_sfa_quant_workspace_bytes(const PtoSfaQuantArgs *a, size_t *bytes)
{
    if (!bytes) return fail(PTO_E_INVALID_ARG, "sfa: bytes is NULL");
    int rc = sfa_check(a);
    if (rc != PTO_OK) return rc;
    const SfaPlan pl = sfa_plan(a);
    *bytes = sfa_ws_bytes(pl);
    return PTO_OK;
}

int pto_sfa_quant_launch(const PtoSfaQuantArgs *a, void *hip_stream)
{
    int rc = sfa_check(a);
    if (rc != PTO_OK) return rc;
    if (!a->query_nope || !a->query_rope || !a->key_nope_2d || !a->key_rope_2d || !a->k_nope_scales || !a->topk_indices ||
        !a->block_table || !a->kv_act_seqs || !a->attention_out)
        return fail(PTO_E_INVALID_ARG, "sfa: a tensor pointer is NULL");
    return sfa_enqueue(a, static_cast<const int8_t *>(a->key_nope_2d), 512, static_cast<const uint8_t *>(a->key_rope_2d), 128,
                       static_cast<const uint8_t *>(a->k_nope_scales), 16, hip_stream);
}

int pto_sfa_quant_launch_static(const PtoSfaQuantArgs *a, void *hip_stream)
{
    int rc = sfa_check(a);
    if (rc != PTO_OK) return rc;
    if (!a->query_nope || !a->query_rope || !a->key_nope_2d || !a->key_rope_2d || !a->k_nope_scales || !a->topk_indices ||
        !a->block_table || !a->kv_act_seqs || !a->attention_out)
        return fail(PTO_E_INVALID_ARG, "sfa: a tensor pointer is NULL");
    const SfaPlan pl = sfa_plan(a, SFA_STATIC_SCRATCH_BYTES);
    const size_t need = sfa_ws_bytes(pl);
    if (need > SFA_STATIC_SCRATCH_BYTES)
        return fail(PTO_E_WORKSPACE,
                    "sfa: the key splits of this shape need %zu bytes of scratch, the built-in array holds %zu; use "
                    "pto_sfa_quant_launch with a workspace, or fewer splits",
                    need, SFA_STATIC_SCRATCH_BYTES);
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(PTO_E_NO_DEVICE, "sfa: no current device: %s", hipGetErrorString(e));
    void *ptr = scratch_of(dev, &e);
    if (!ptr) return fail(PTO_E_NO_DEVICE, "sfa: the scratch array has no address on device %d: %s", dev, hipGetErrorString(e));
    PtoSfaQuantArgs q = *a;
    q.workspace = ptr;
    q.workspace_bytes = SFA_STATIC_SCRATCH_BYTES;
    return sfa_enqueue(&q, static_cast<const int8_t *>(a->key_nope_2d), 512, static_cast<const uint8_t *>(a->key_rope_2d), 128,
                       static_cast<const uint8_t *>(a->k_nope_scales), 16, hip_stream, false, SFA_STATIC_SCRATCH_BYTES);
}

int pto_sfa_bf16kv_launch(const PtoSfaQuantArgs *a, void *hip_stream)
{
    int rc = sfa_check(a);
    if (rc != PTO_OK) return rc;
    if (!a->query_nope || !a->query_rope || !a->key_nope_2d || !a->key_rope_2d || !a->topk_indices || !a->block_table ||
        !a->kv_act_seqs || !a->attention_out)
        return fail(PTO_E_INVALID_ARG, "sfa: a tensor pointer is NULL");
    return sfa_enqueue(a, static_cast<const int8_t *>(a->key_nope_2d), 1024, static_cast<const uint8_t *>(a->key_rope_2d), 128,
                       static_cast<const uint8_t *>(a->key_nope_2d), 0, hip_stream, true);
}

int pto_sa_antiquant_workspace_bytes(const PtoSaAntiquantArgs *a, size_t *bytes)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "sfa: args is NULL");
    const PtoSfaQuantArgs q = unpacked_view(a);
    return pto_sfa_quant_workspace_bytes(&q, bytes);
}

int pto_sa_antiquant_launch(const PtoSaAntiquantArgs *a, void *hip_stream)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "sfa: args is NULL");
    const PtoSfaQuantArgs q = unpacked_view(a);
    int rc = sfa_check(&q);
    if (rc != PTO_OK) return rc;
    if (!a->query_nope || !a->query_rope || !a->nope_cache || !a->topk_indices || !a->block_table || !a->kv_act_seqs ||
        !a->attention_out)
        return fail(PTO_E_INVALID_ARG, "sfa: a tensor pointer is NULL");
    const uint8_t *base = static_cast<const uint8_t *>(a->nope_cache);
    return sfa_enqueue(&q, reinterpret_cast<const int8_t *>(base), PACKED_ROW_BYTES, base + 512, PACKED_ROW_BYTES, base + 640,
                       PACKED_ROW_BYTES, hip_stream);
}

int pto_li_decode_workspace_bytes(const PtoLiDecodeArgs *a, size_t *bytes)
{
    if (!bytes) return fail(PTO_E_INVALID_ARG, "li: bytes is NULL");
    int rc = li_check(a);
    if (rc != PTO_OK) return rc;
    *bytes = li_ws_bytes(a);
    return PTO_OK;
}

int pto_li_decode_launch(const PtoLiDecodeArgs *a, void *hip_stream)
{
    int rc = li_check(a);
    if (rc != PTO_OK) return rc;
    if (!a->idx_query || !a->idx_query_scale || !a->idx_key_cache || !a->idx_key_scale || !a->idx_weight || !a->act_seq_key ||
        !a->block_table || !a->topk_res)
        return fail(PTO_E_INVALID_ARG, "li: a tensor pointer is NULL");
    const size_t need = li_ws_bytes(a);
    if (!a->workspace || a->workspace_bytes < need)
        return fail(PTO_E_WORKSPACE, "li: workspace of %zu bytes required, %zu given", need, a->workspace ? a->workspace_bytes : (size_t)0);
    if (cu_count() <= 0) return fail(PTO_E_NO_DEVICE, "li: no usable device is current");
    {
        const void *al16[] = {a->idx_query, a->idx_key_cache, a->workspace};
        for (const void *ptr : al16)
            if (reinterpret_cast<uintptr_t>(ptr) & 15)
                return fail(PTO_E_INVALID_ARG, "li: query, key-cache and workspace pointers must be 16-byte aligned");
        const void *al4[] = {a->act_seq_key, a->block_table, a->topk_res};
        for (const void *ptr : al4)
            if (reinterpret_cast<uintptr_t>(ptr) & 3)
                return fail(PTO_E_INVALID_ARG, "li: length, block-table and result pointers must be 4-byte aligned");
        const void *sc[] = {a->idx_query_scale, a->idx_key_scale, a->idx_weight};
        const int sdt[] = {a->q_scale_dtype, a->k_scale_dtype, a->weight_dtype};
        for (int i = 0; i < 3; ++i)
            if (reinterpret_cast<uintptr_t>(sc[i]) & (sdt[i] == PTO_DT_FP32 ? 3 : 1))
                return fail(PTO_E_INVALID_ARG, "li: scale and weight pointers must be aligned to their element size");
    }

    pto::LiParams p;
    p.q = a->idx_query;
    p.q_scale = a->idx_query_scale;
    p.kcache = a->idx_key_cache;
    p.k_scale = a->idx_key_scale;
    p.weight = a->idx_weight;
    p.act = a->act_seq_key;
    p.bt = a->block_table;
    p.topk_res = a->topk_res;
    p.T = (int)a->t;
    p.B = (int)a->b;
    p.S1 = (int)(a->t / a->b);
    p.bs = (int)a->block_size;
    p.maxblk = (int)a->max_blocknum_perbatch;
    p.nblocks = (int)a->block_num;
    p.k = (int)a->selected_count;
    p.score_stride = (long long)a->max_blocknum_perbatch * a->block_size;
    p.scores = static_cast<float *>(a->workspace);
    p.sample = p.scores + (size_t)a->t * p.score_stride;
    p.q_dt = a->q_scale_dtype;
    p.k_dt = a->k_scale_dtype;
    p.w_dt = a->weight_dtype;
    p.variant = a->arith_variant;
    {   // A wave pays three dependent memory latencies before its first pair, so runs are made as long
        // as still leaves every SIMD two rounds of two waves; at most 32 pairs (2048 keys) per wave.
        // Two query tokens of a sequence share a key pass (half the key bytes, the same arithmetic) when
        // there are two and the pass then still has several rounds of work for every resident wave; a
        // small batch is bound by latency, not bytes, and keeps one token per wave for twice the waves.
        int nt = 1;
        if (p.S1 >= 2 && p.variant == 0) {
            const long long pairs2 = (long long)p.B * ((p.S1 + 1) / 2) * ((p.score_stride + 63) / 64);
            if (pairs2 >= 8ll * cu_count() * 8) nt = 2;
        }
        p.nt = nt;
        const long long units = (long long)p.B * ((p.S1 + nt - 1) / nt);    // token groups that share a key pass
        const long long pairs = units * ((p.score_stride + 63) / 64);
        long long ppw = pairs / ((long long)cu_count() * 4 * 4);
        p.ppw = (int)(ppw < 1 ? 1 : (ppw > pto::LI_MAX_PAIRS_PER_WAVE ? pto::LI_MAX_PAIRS_PER_WAVE : ppw));
        // With few units the kernel balances the runs itself from the actual lengths: one round
        // of resident waves (two workgroups per CU), more only if the longest possible input needs it.
        p.balanced = units <= pto::LI_MAX_BALANCED_TOKENS;
        long long waves = (long long)cu_count() * 8;
        const long long need = (pairs + pto::LI_MAX_PAIRS_PER_WAVE - 1) / pto::LI_MAX_PAIRS_PER_WAVE + 2 * units;
        waves = waves > need ? waves : need;
        p.score_wgs = (int)((waves + 3) / 4);
    }
    hipError_t e = pto::li_launch(p, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_E_LAUNCH, "li: launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

int pto_li_prolog_quant_workspace_bytes(const PtoLiPrologQuantArgs *a, size_t *bytes)
{
    if (!bytes) return fail(PTO_E_INVALID_ARG, "li_prolog: bytes is NULL");
    int rc = lip_check(a);
    if (rc != PTO_OK) return rc;
    *bytes = lip_ws_bytes(a);
    return PTO_OK;
}

// checked arguments -> kernel parameters
static int lip_params(const PtoLiPrologQuantArgs *a, pto::LipParams &p)
{
    if (a && (a->sum_mode < 0 || a->sum_mode > 2)) return fail(PTO_E_INVALID_ARG, "li_prolog: sum_mode must be 0, 1 or 2");
    int rc = lip_check(a);
    if (rc != PTO_OK) return rc;
    if (!a->x || !a->q_norm || !a->q_norm_scale || !a->w_qb || !a->w_qb_scale || !a->wk || !a->w_proj || !a->ln_gamma_k ||
        !a->ln_beta_k || !a->cos_idx_rope || !a->sin_idx_rope || !a->hadamard_q || !a->hadamard_k || !a->k_cache ||
        !a->k_cache_scale || !a->k_cache_index || !a->q_int8 || !a->q_scale || !a->weights)
        return fail(PTO_E_INVALID_ARG, "li_prolog: a tensor pointer is NULL");
    const size_t need = lip_ws_bytes(a);
    if (!a->workspace || a->workspace_bytes < need)
        return fail(PTO_E_WORKSPACE, "li_prolog: workspace of %zu bytes required, %zu given", need,
                    a->workspace ? a->workspace_bytes : (size_t)0);
    const void *aligned[] = {a->x, a->q_norm, a->q_norm_scale, a->w_qb, a->w_qb_scale, a->wk, a->w_proj, a->ln_gamma_k, a->ln_beta_k,
                             a->cos_idx_rope, a->sin_idx_rope, a->hadamard_q, a->hadamard_k, a->k_cache, a->q_int8, a->workspace};
    for (const void *ptr : aligned)
        if (reinterpret_cast<uintptr_t>(ptr) & 15)
            return fail(PTO_E_INVALID_ARG, "li_prolog: tensor and workspace pointers must be 16-byte aligned");

    p.x = static_cast<const uint16_t *>(a->x);
    p.q_norm = a->q_norm;
    p.q_norm_scale = a->q_norm_scale;
    p.w_qb = a->w_qb;
    p.w_qb_scale = a->w_qb_scale;
    p.wk = static_cast<const uint16_t *>(a->wk);
    p.w_proj = static_cast<const uint16_t *>(a->w_proj);
    p.gamma = static_cast<const uint16_t *>(a->ln_gamma_k);
    p.beta = static_cast<const uint16_t *>(a->ln_beta_k);
    p.cos = static_cast<const uint16_t *>(a->cos_idx_rope);
    p.sin = static_cast<const uint16_t *>(a->sin_idx_rope);
    p.hq = static_cast<const uint16_t *>(a->hadamard_q);
    p.hk = static_cast<const uint16_t *>(a->hadamard_k);
    p.k_cache = a->k_cache;
    p.k_cache_scale = static_cast<uint16_t *>(a->k_cache_scale);
    p.k_cache_index = reinterpret_cast<const long long *>(a->k_cache_index);
    p.q_int8 = a->q_int8;
    p.q_scale = static_cast<uint16_t *>(a->q_scale);
    p.weights = static_cast<uint16_t *>(a->weights);
    p.qpart = static_cast<int32_t *>(a->workspace);
    p.xpart = reinterpret_cast<float *>(static_cast<char *>(a->workspace) + lip_qpart_bytes(a));
    p.cache_rows = a->cache_rows;
    p.T = (int)a->t;
    p.h = (int)a->h;
    p.q_lora = (int)a->q_lora_rank;
    p.n_heads = (int)a->n_heads;
    p.eps = a->eps;
    p.sum_mode = a->sum_mode;
    p.x_in_groups = 0;
    p.w_mul0 = (float)std::pow((double)a->n_heads, -0.5);
    p.w_mul1 = (float)std::pow((double)pto::LIP_DIM, -0.5);
    return PTO_OK;
}

int pto_li_prolog_quant_launch(const PtoLiPrologQuantArgs *a, void *hip_stream)
{
    pto::LipParams p;
    int rc = lip_params(a, p);
    if (rc != PTO_OK) return rc;
    hipError_t e = pto::lip_launch(p, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_E_LAUNCH, "li_prolog: launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

int pto_mla_prolog_quant_workspace_bytes(const PtoMlaPrologQuantArgs *a, size_t *bytes)
{
    if (!bytes) return fail(PTO_E_INVALID_ARG, "mla_prolog: bytes is NULL");
    int rc = mlap_check(a);
    if (rc != PTO_OK) return rc;
    *bytes = mlap_ws_bytes(a);
    return PTO_OK;
}

// checked arguments -> kernel parameters
static int mlap_params(const PtoMlaPrologQuantArgs *a, pto::MlapParams &p)
{
    int rc = mlap_check(a);
    if (rc != PTO_OK) return rc;
    const void *ptrs[] = {a->token_x, a->w_dq, a->w_uq_qr, a->dequant_scale, a->w_uk, a->w_dkv_kr, a->gamma_cq, a->gamma_ckv,
                          a->cos, a->sin, a->cache_index, a->kv_cache, a->kr_cache, a->k_scale_cache, a->q_norm_out,
                          a->q_norm_scale_out, a->query_nope_out, a->query_rope_out};
    for (const void *ptr : ptrs)
        if (!ptr) return fail(PTO_E_INVALID_ARG, "mla_prolog: a tensor pointer is NULL");
    const size_t need = mlap_ws_bytes(a);
    if (!a->workspace || a->workspace_bytes < need)
        return fail(PTO_E_WORKSPACE, "mla_prolog: workspace of %zu bytes required, %zu given", need,
                    a->workspace ? a->workspace_bytes : (size_t)0);
    const void *aligned[] = {a->token_x, a->w_dq, a->w_uq_qr, a->dequant_scale, a->w_uk, a->w_dkv_kr, a->gamma_cq, a->gamma_ckv,
                             a->kv_cache, a->k_scale_cache, a->q_norm_out, a->workspace};
    for (const void *ptr : aligned)
        if (reinterpret_cast<uintptr_t>(ptr) & 15)
            return fail(PTO_E_INVALID_ARG, "mla_prolog: tensor and workspace pointers must be 16-byte aligned");

    p.x = static_cast<const uint16_t *>(a->token_x);
    p.w_dq = static_cast<const uint16_t *>(a->w_dq);
    p.w_uqqr = a->w_uq_qr;
    p.w_qb_scale = a->dequant_scale;
    p.w_uk = static_cast<const uint16_t *>(a->w_uk);
    p.w_dkvkr = static_cast<const uint16_t *>(a->w_dkv_kr);
    p.gamma_cq = static_cast<const uint16_t *>(a->gamma_cq);
    p.gamma_ckv = static_cast<const uint16_t *>(a->gamma_ckv);
    p.cos = static_cast<const uint16_t *>(a->cos);
    p.sin = static_cast<const uint16_t *>(a->sin);
    p.cache_index = reinterpret_cast<const long long *>(a->cache_index);
    p.kv_cache = a->kv_cache;
    p.kr_cache = static_cast<uint16_t *>(a->kr_cache);
    p.k_scale_cache = a->k_scale_cache;
    p.q_norm = a->q_norm_out;
    p.q_norm_scale = a->q_norm_scale_out;
    p.q_nope = static_cast<uint16_t *>(a->query_nope_out);
    p.q_rope = static_cast<uint16_t *>(a->query_rope_out);
    p.xpart = static_cast<float *>(a->workspace);
    p.qpart = reinterpret_cast<int32_t *>(static_cast<char *>(a->workspace) + mlap_xpart_bytes(a));
    p.cache_rows = a->cache_rows;
    p.T = (int)a->t;
    p.h = (int)a->h;
    p.q_lora = (int)a->q_lora_rank;
    p.n_heads = (int)a->n_heads;
    p.eps_cq = a->epsilon_cq;
    p.eps_ckv = a->epsilon_ckv;
    p.absorb_exact = a->absorb_exact ? 1 : 0;
    return PTO_OK;
}

int pto_mla_prolog_quant_launch(const PtoMlaPrologQuantArgs *a, void *hip_stream)
{
    pto::MlapParams p;
    int rc = mlap_params(a, p);
    if (rc != PTO_OK) return rc;
    hipError_t e = pto::mlap_launch(p, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_E_LAUNCH, "mla_prolog: launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

// ---- both prologs as one operator: the query latent and its scale live in the common workspace

namespace {

struct FusedPlan {
    size_t q_norm_off, q_norm_scale_off, rest_off, total;
    PtoMlaPrologQuantArgs mla;
    PtoLiPrologQuantArgs idx;
};

// fills in what the two halves share and where the intermediates go (workspace base may be null: sizes only)
int fused_plan(const PtoMlaIndexerPrologQuantArgs *a, FusedPlan *pl)
{
    if (!a) return fail(PTO_E_INVALID_ARG, "mla_indexer_prolog: args is NULL");
    pl->mla = a->mla;
    pl->idx = a->indexer;
    pl->idx.x = a->mla.token_x;
    pl->idx.cos_idx_rope = a->mla.cos;
    pl->idx.sin_idx_rope = a->mla.sin;
    pl->idx.k_cache_index = a->mla.cache_index;
    pl->idx.t = a->mla.t;
    pl->idx.h = a->mla.h;
    pl->idx.q_lora_rank = a->mla.q_lora_rank;
    int rc = mlap_check(&pl->mla);
    if (rc != PTO_OK) return rc;
    rc = lip_check(&pl->idx);
    if (rc != PTO_OK) return rc;
    const size_t qn = ((size_t)a->mla.t * a->mla.q_lora_rank + 255) & ~(size_t)255;
    const size_t qs = ((size_t)a->mla.t * sizeof(float) + 255) & ~(size_t)255;
    const size_t w_mla = mlap_ws_bytes(&pl->mla), w_idx = lip_ws_bytes(&pl->idx);
    pl->q_norm_off = 0;
    pl->q_norm_scale_off = qn;
    pl->rest_off = qn + qs;
    // the partial sums of both halves are alive at once (the last launch finishes both), so each has its own area
    const size_t w_mla_pad = (w_mla + 255) & ~(size_t)255;
    pl->total = qn + qs + w_mla_pad + w_idx;
    char *base = static_cast<char *>(a->workspace);
    if (base) {
        int8_t *q_norm = a->mla.q_norm_out ? a->mla.q_norm_out : reinterpret_cast<int8_t *>(base + pl->q_norm_off);
        float *q_norm_scale = a->mla.q_norm_scale_out ? a->mla.q_norm_scale_out : reinterpret_cast<float *>(base + pl->q_norm_scale_off);
        pl->mla.q_norm_out = q_norm;
        pl->mla.q_norm_scale_out = q_norm_scale;
        pl->idx.q_norm = q_norm;
        pl->idx.q_norm_scale = q_norm_scale;
        pl->mla.workspace = base + pl->rest_off;
        pl->mla.workspace_bytes = w_mla;
        pl->idx.workspace = base + pl->rest_off + w_mla_pad;
        pl->idx.workspace_bytes = w_idx;
    }
    return PTO_OK;
}

}  // namespace

int pto_mla_indexer_prolog_quant_workspace_bytes(const PtoMlaIndexerPrologQuantArgs *a, size_t *bytes)
{
    if (!bytes) return fail(PTO_E_INVALID_ARG, "mla_indexer_prolog: bytes is NULL");
    FusedPlan pl;
    int rc = fused_plan(a, &pl);
    if (rc != PTO_OK) return rc;
    *bytes = pl.total;
    return PTO_OK;
}

int pto_mla_indexer_prolog_quant_launch(const PtoMlaIndexerPrologQuantArgs *a, void *hip_stream)
{
    FusedPlan pl;
    int rc = fused_plan(a, &pl);
    if (rc != PTO_OK) return rc;
    if (!a->workspace || a->workspace_bytes < pl.total)
        return fail(PTO_E_WORKSPACE, "mla_indexer_prolog: workspace of %zu bytes required, %zu given", pl.total,
                    a->workspace ? a->workspace_bytes : (size_t)0);
    if (reinterpret_cast<uintptr_t>(a->workspace) & 255)
        return fail(PTO_E_INVALID_ARG, "mla_indexer_prolog: the workspace must be 256-byte aligned");
    pto::MlapParams pm;
    pto::LipParams pi;
    rc = mlap_params(&pl.mla, pm);
    if (rc != PTO_OK) return rc;
    rc = lip_params(&pl.idx, pi);
    if (rc != PTO_OK) return rc;
    // four launches up to 32 tokens (the indexer half rides in the MLA half's), five up to 63, six above
    hipError_t e = pto::prolog_fused_launch(pm, pi, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(PTO_E_LAUNCH, "mla_indexer_prolog: launch failed: %s", hipGetErrorString(e));
    return PTO_OK;
}

}  // extern "C"
