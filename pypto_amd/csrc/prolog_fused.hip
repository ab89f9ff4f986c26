// MLA prolog + lightning-indexer prolog as one operator (mla_indexer_prolog_quant_d/_p of the reference,
// examples/models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:141-256).  At decode sizes it is the MLA
// prolog's four launches with the indexer prolog's work riding in them (MlapRider): hidden-axis sums (wk as one
// more column slab, w_proj beside the rope columns of w_dkv_kr) -> norms and quantisation of the latents -> int8
// projections of the attention query and of the indexer query, jobs of one kind -> ONE last launch for both: the
// workgroups that finish the attention query (absorb product, 70 KB of LDS, four waves) and those that finish the
// indexer's query rows, key row and weights (54 KB, eight waves) do not depend on each other and fit a compute
// unit together, so they run side by side instead of one launch after the other.  Where the indexer prolog cannot
// ride (other than 64 indexer heads) its first launch follows the MLA prolog's third.  Between 9 and 63 tokens the
// MLA prolog's prefill forms take the jobs of the indexer prolog's first launch along as riders (five launches;
// four up to 32 tokens, where the two last stages share one); from 64 tokens on every stage has a launch of its own.
#include "prolog_finish.h"

#include "prolog_fused.h"

namespace pto {
namespace {

constexpr int FUSED_FIN_LDS = MLAP_FIN_LDS > LIP_FIN_LDS ? MLAP_FIN_LDS : LIP_FIN_LDS;
static_assert(2 * FUSED_FIN_LDS <= 160 * 1024, "two workgroups of the last launch share a compute unit");

// Workgroups [0, mla_wgs): the MLA prolog's last launch (its 256 threads; the other four waves pass the body's
// barriers with them and leave).  The rest: the indexer prolog's second launch.
__global__ __launch_bounds__(64 * FIN_WAVES) void prolog_fused_finish_kernel(const MlapParams pm, const LipParams pl, const int mla_wgs,
                                                                             const int q_wgs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[FUSED_FIN_LDS];
    if ((int)blockIdx.x < mla_wgs) {
        if (threadIdx.x >= 256) {
            for (int i = 0; i < MLAP_FIN_BARRIERS; ++i) __syncthreads();
            return;
        }
        mlap_finish_body(pm, (int)blockIdx.x, lds);
    } else {
        lip_finish_body(pl, q_wgs, (int)blockIdx.x - mla_wgs, lds);
    }
}

// The same for the MLA prolog's prefill form of its last stage (eight waves like the indexer prolog's, all of a
// compute unit's LDS): between 9 and 32 tokens that form has one workgroup per head -- half of the compute
// units -- and the indexer prolog's workgroups take the compute units it leaves, then the ones it frees, instead of
// waiting for a launch of their own.
constexpr int FUSED_FINP_LDS = MLAP_FINP_LDS > LIP_FIN_LDS ? MLAP_FINP_LDS : LIP_FIN_LDS;
static_assert(FINP_WAVES == FIN_WAVES, "one block size for both bodies");
__global__ __launch_bounds__(64 * FIN_WAVES) void prolog_fused_finish_prefill_kernel(const MlapParams pm, const int per, const LipParams pl,
                                                                                     const int mla_wgs, const int q_wgs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[FUSED_FINP_LDS];
    if ((int)blockIdx.x < mla_wgs) mlap_finish_prefill_body(pm, (int)blockIdx.x, per, lds);
    else lip_finish_body(pl, q_wgs, (int)blockIdx.x - mla_wgs, lds);
}

}  // namespace

hipError_t prolog_fused_launch(const MlapParams &pm, const LipParams &pl, hipStream_t stream)
{
    // Decode sizes: the indexer prolog's first launch has no work of a kind of its own -- its sums over the hidden
    // axis are more column slabs of the MLA prolog's first launch and its int8 projection more jobs of the third
    // (MlapRider) -- so the pass is four launches: hidden-axis sums, latents, projections, one finish for both.
    if (mlap_takes_rider(pm) && pl.T == pm.T && pl.h == pm.h && pl.q_lora == pm.q_lora && pl.x == pm.x && pl.q_norm == pm.q_norm &&
        pl.q_norm_scale == pm.q_norm_scale && pl.n_heads == 64 && !lip_q_on_matrix_cores(pl)) {
        const MlapRider rd = {pl.wk, pl.w_proj, pl.xpart, pl.w_qb, pl.qpart, pl.n_heads};
        hipError_t e = mlap_launch_front(pm, stream, &rd);
        if (e != hipSuccess) return e;
        LipParams pg = pl;
        pg.x_in_groups = 1;
        const int mla_wgs = mlap_finish_wgs(pm);
        const int q_wgs = lip_finish_query_wgs(pg);
        hipLaunchKernelGGL(prolog_fused_finish_kernel, dim3((unsigned)(mla_wgs + q_wgs + pg.T)), dim3(64 * FIN_WAVES), 0, stream, pm, pg,
                           mla_wgs, q_wgs);
        return hipGetLastError();
    }
    // A batch of 9 to 63 tokens: the MLA prolog runs its prefill forms, the indexer prolog its decode forms, and the
    // jobs of the indexer prolog's first launch (wave jobs with no kind of workgroup of their own) ride in the MLA
    // prolog's first and third launch, whose workgroups leave half of every compute unit free, and up to 32 tokens the
    // finishing stages of the two halves share the last launch: four launches, five above.
    const bool lip_rides = mlap_takes_lip_rider(pm) && pl.T == pm.T && pl.h == pm.h && pl.q_lora == pm.q_lora && pl.x == pm.x &&
                           pl.q_norm == pm.q_norm && pl.q_norm_scale == pm.q_norm_scale && !lip_q_on_matrix_cores(pl) &&
                           !lip_x_on_matrix_cores(pl) && !lip_x_group_rows(pl) && pl.n_heads <= LIP_MAX_HEADS;
    hipError_t e = mlap_launch_front(pm, stream, nullptr, lip_rides ? &pl : nullptr);
    if (e != hipSuccess) return e;
    if (!lip_rides) {
        e = lip_launch_linear(pl, stream);
        if (e != hipSuccess) return e;
    }
    int per = 0, pf_wgs = 0;
    if (mlap_finish_is_prefill(pm)) mlap_finish_prefill_shape(pm, per, pf_wgs);
    // up to 32 tokens: one workgroup per head, the indexer half's take the other compute units (more would queue one
    // to a compute unit behind a full chip, slower than their own launch at two)
    if (mlap_finish_is_prefill(pm) && !lip_q_on_matrix_cores(pl) && pf_wgs <= 128) {
        const int q_wgs = lip_finish_query_wgs(pl);
        hipLaunchKernelGGL(prolog_fused_finish_prefill_kernel, dim3((unsigned)(pf_wgs + q_wgs + pl.T)), dim3(64 * FIN_WAVES), 0, stream, pm, per,
                           pl, pf_wgs, q_wgs);
        return hipGetLastError();
    }
    if (mlap_finish_is_prefill(pm) || lip_q_on_matrix_cores(pl)) {
        // prefill sizes: the last stages have forms of their own (the attention query's: one workgroup per compute unit)
        e = mlap_launch_finish(pm, stream);
        if (e != hipSuccess) return e;
        return lip_launch_finish(pl, stream);
    }
    const int mla_wgs = mlap_finish_wgs(pm);
    const int q_wgs = lip_finish_query_wgs(pl);
    hipLaunchKernelGGL(prolog_fused_finish_kernel, dim3((unsigned)(mla_wgs + q_wgs + pl.T)), dim3(64 * FIN_WAVES), 0, stream, pm, pl,
                       mla_wgs, q_wgs);
    return hipGetLastError();
}

}  // namespace pto
