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
// Two launches; below LIP_MFMA_MIN_TOKENS tokens (decode):
//   lip_linear_kernel   workgroups of four independent waves.  Two of them share a query job (head,
//                       quarter of the reduction axis, block of 32 tokens), one half each: the tile of
//                       w_qb (rows x 128 bytes) and the token rows travel to LDS by LDS-DMA, all
//                       requests issued up front; 32-row steps are consumed as their requests land
//                       (they complete in order): the transposing 8-bit LDS read (ds_read_b64_tr_b8, two per
//                       product) turns the row-major tile into v_mfma_i32_32x32x32_i8 operands.  The two halves are added through
//                       LDS and the partial int32 sums go to the workspace.  The other two waves take
//                       hidden-axis jobs (block of 64 rows of wk or of w_proj, 4 tokens): fp32 FMAs
//                       with the hidden states as scalar operands; block sums go to the workspace.
//   lip_finish_kernel   Query rows, one per wave: add the four partial sums, de-quantise, rope,
//                       Hadamard (matrix staged in LDS once per workgroup), quantise, store.  Tokens,
//                       one workgroup each: waves add the groups of block sums, then one wave finishes
//                       the key row (layer norm, rope, Hadamard, quantise, scatter) and one the weights.
// From LIP_MFMA_MIN_TOKENS tokens on (prefill chunks) the stages take forms of their own (LipParams::sum_mode says
// which sums may leave their fixed order):
//   lip_qproj_prefill_kernel, lip_qproj_prefill256_kernel   the query projection unsplit (prolog_common.h), a
//                       workgroup per 128 x 128 or 256 x 256 tile over the whole reduction axis; exact.
//   lip_xlinear_group_kernel   the fixed-order sums over the hidden axis, a group of eight blocks per workgroup and 16
//                       tokens per weight block, hidden states broadcast by DPP (xlinear_fixed.h); or
//   lip_xlinear_mfma_kernel    the same sums on the matrix cores (xlinear_mfma.h), if asked for.
//   lip_finish_query_prefill_kernel   query rows with the Hadamard sums on the matrix cores, 32 rows per pass of a
//                       wave (prolog_finish.h), unless every sum is to keep its fixed order.
//   lip_finish_tokens_prefill_kernel  key rows and weights, eight tokens per workgroup.
#include "lip_kernels.h"
#include "prolog_common.h"
#include "prolog_finish.h"
#include "lip_xjob.h"
#include "xlinear_fixed.h"
#include "xlinear_mfma.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

static_assert(LIP_KSPLIT == QPROJ_KSPLIT, "workspace sizing and the projection job disagree");

// ---------------------------------------------------------------------------------------------
// Hidden-axis jobs: lip_xjob.h.
template <int HS>
constexpr int lin_lds_bytes()
{
    return 2 * lin_region_bytes<HS>() + LIN_XWAVES * X_REGION_BYTES;
}

// Workgroup of six waves, no dependencies among them except the final pairwise sum of the two query
// waves: waves 0 and 1 run the two halves of query job blockIdx.x, waves 2..5 walk the hidden-axis jobs.
template <int HS, int XTOK>
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

    const QProj qp = {p.q_norm, p.w_qb, p.qpart, p.T, p.q_lora, p.n_heads, p.q_norm_scale, p.w_qb_scale};
    if (qwave) {
        q_half_job<HS>(qp, region, job, w, acc);
        if (w == 1) q_pair_park(region, l, acc);
    } else if (w >= 2) {
        uint8_t *xregion = lip_smem + 2 * lin_region_bytes<HS>() + (w - 2) * X_REGION_BYTES;
        for (int j = job * LIN_XWAVES + (w - 2); j < x_jobs; j += gridDim.x * LIN_XWAVES) x_linear_job<XTOK>(p, xregion, j);
    }
    __syncthreads();
    if (qwave && w == 0) q_pair_store<HS>(qp, lip_smem, job, l, acc);
}

template <int TB>
__global__ __launch_bounds__(256) void lip_qproj_prefill_kernel(const QProj p, const int njobs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[QPF_LDS];
    q_prefill_body<TB>(p, q_prefill_job_of((int)blockIdx.x, njobs), lds);
}

// The fixed-order sums over the hidden axis at prefill sizes (xlinear_fixed.h, the form that broadcasts the hidden
// states through DPP): workgroup = (wk or w_proj, group of eight blocks, 16 tokens); only the group sums reach memory,
// an eighth of the rows the decode form leaves, and a block of weights serves sixteen tokens instead of two.
static_assert(XL_BLOCK == LIP_XBLOCK && XL_GROUP == LIP_XGROUP, "the second launch adds groups of eight blocks of 64");
__global__ __launch_bounds__(64 * XL_WAVES) void lip_xlinear_group_kernel(const LipParams p, const int ngroups)
{
    __shared__ __attribute__((aligned(16))) uint8_t smem[XD_LDS];
    const int slab = blockIdx.x & 1;
    const int g = (blockIdx.x >> 1) % ngroups;
    const int t0 = ((blockIdx.x >> 1) / ngroups) * XD_TOK;
    XlSlab sl;
    sl.w = reinterpret_cast<const uint8_t *>(slab ? p.w_proj : p.wk);
    sl.pitch = (slab ? p.n_heads : LIP_DIM) * 2;
    sl.wbytes = sl.pitch;
    sl.out = p.xpart + (size_t)g * p.T * LIP_XCOLS + slab * LIP_DIM;
    sl.out_pitch = LIP_XCOLS;
    if (slab) xd_body<false>(sl, p.x, p.T, p.h, g, t0, smem);      // w_proj: one column per lane
    else xd_body<true>(sl, p.x, p.T, p.h, g, t0, smem);
}

// The sums over the hidden axis on the matrix cores (xlinear_mfma.h): workgroup = (wk or w_proj, one of nsplit
// ranges of the hidden axis, 128 tokens); w_proj is a narrow slab of n_heads columns.
static_assert(XM_KC == LIP_XBLOCK, "the workspace is sized in chunks of the hidden axis");
__global__ __launch_bounds__(256) void lip_xlinear_mfma_kernel(const LipParams p, const int nsplit)
{
    __shared__ __attribute__((aligned(16))) uint8_t smem[XM_LDS];
    const int slab = blockIdx.x & 1;
    const int sp = (blockIdx.x >> 1) % nsplit;
    const int t0 = ((blockIdx.x >> 1) / nsplit) * XM_TOK;
    XmSlab sl;
    sl.w = reinterpret_cast<const uint8_t *>(slab ? p.w_proj : p.wk);
    sl.pitch = (slab ? p.n_heads : LIP_DIM) * 2;
    sl.pieces = slab ? p.n_heads / 8 : 16;
    sl.out = p.xpart + (size_t)sp * p.T * LIP_XCOLS + slab * LIP_DIM;
    sl.out_pitch = LIP_XCOLS;
    const int nchunks = p.h / XM_KC;
    xm_body(sl, p.x, p.T, p.h, t0, (int)((long long)sp * nchunks / nsplit), (int)((long long)(sp + 1) * nchunks / nsplit), smem);
}

__global__ __launch_bounds__(64 * QFP_WAVES) void lip_finish_query_prefill_kernel(const LipParams p)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[LIP_QFP_LDS];
    lip_finish_query_prefill_body(p, (int)blockIdx.x, (int)gridDim.x, lds);
}

__global__ __launch_bounds__(512) void lip_qproj_prefill256_kernel(const QProj p, const int njobs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[QP2_LDS];
    q_prefill256_body(p, q_prefill_job_of((int)blockIdx.x, njobs), lds);
}

__global__ __launch_bounds__(64 * FIN_WAVES) void lip_finish_tokens_prefill_kernel(const LipParams p)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[LIP_FINT_LDS];
    lip_finish_tokens_prefill_body(p, (int)blockIdx.x, lds);
}

// ---------------------------------------------------------------------------------------------
// Second launch: prolog_finish.h.
__global__ __launch_bounds__(64 * FIN_WAVES) void lip_finish_kernel(const LipParams p, const int q_wgs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[LIP_FIN_LDS];
    lip_finish_body(p, q_wgs, (int)blockIdx.x, lds);
}

}  // namespace

// workgroups of the second launch that finish query rows (none where the rows have a launch of their own)
int lip_finish_query_wgs(const LipParams &p) { return lip_q_on_matrix_cores(p) ? 0 : (p.T * p.n_heads + FIN_WAVES - 1) / FIN_WAVES; }

hipError_t lip_launch_linear(const LipParams &p, hipStream_t stream)
{
    const int steps = p.q_lora / LIP_KSPLIT / 32;
    const int tblocks = (p.T + 31) / 32;
    const bool unsplit = qproj_splits(p.T) == 1;      // prefill sizes: the query projection as a launch of its own
    const int q_jobs = unsplit ? 0 : p.n_heads * LIP_KSPLIT * tblocks;
    if (unsplit) {
        if (p.q_lora % (32 * QPF_STEPS)) return hipErrorInvalidValue;
        const QProj qp = {p.q_norm, p.w_qb, p.qpart, p.T, p.q_lora, p.n_heads, p.q_norm_scale, p.w_qb_scale};
        const int cus = cu_count();
        if (cus <= 0) return hipErrorNoDevice;
        const int njobs256 = q_prefill256_jobs(qp);
        if (4 * njobs256 >= 3 * cus) {                // enough 256 x 256 tiles to fill the chip
            hipLaunchKernelGGL(lip_qproj_prefill256_kernel, dim3((unsigned)njobs256), dim3(512), 0, stream, qp, njobs256);
        } else {
            const int njobs = q_prefill_jobs(qp);
            const dim3 g((unsigned)njobs), b(256);
            if (q_prefill_token_blocks(p.T) == 2) hipLaunchKernelGGL(lip_qproj_prefill_kernel<2>, g, b, 0, stream, qp, njobs);
            else hipLaunchKernelGGL(lip_qproj_prefill_kernel<4>, g, b, 0, stream, qp, njobs);
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (lip_x_on_matrix_cores(p)) {
        const int nsplit = lip_xrows(p);
        const int ttiles = (p.T + XM_TOK - 1) / XM_TOK;
        hipLaunchKernelGGL(lip_xlinear_mfma_kernel, dim3((unsigned)(2 * nsplit * ttiles)), dim3(256), 0, stream, p, nsplit);
        return hipGetLastError();
    }
    if (lip_x_group_rows(p)) {
        const int ngroups = lip_xrows(p);
        const int tgroups = (p.T + XD_TOK - 1) / XD_TOK;
        hipLaunchKernelGGL(lip_xlinear_group_kernel, dim3((unsigned)(2 * ngroups * tgroups)), dim3(64 * XL_WAVES), 0, stream, p, ngroups);
        return hipGetLastError();
    }
    const int xtok = lip_xtok(p.T);
    const int x_jobs = lip_x_jobs(p, xtok);
    // enough workgroups that each hidden-axis wave gets about one job, never fewer than the query jobs
    int wgs = (x_jobs + LIN_XWAVES - 1) / LIN_XWAVES;
    wgs = wgs > 4096 ? 4096 : wgs;
    wgs = wgs > q_jobs ? wgs : q_jobs;
    const dim3 grid1((unsigned)wgs), block1(128 + 64 * LIN_XWAVES);
#define LIP_LINEAR(HS)                                                                                              \
    switch (xtok) {                                                                                                \
    case 2: hipLaunchKernelGGL((lip_linear_kernel<HS, 2>), grid1, block1, 0, stream, p, q_jobs, x_jobs); break;  \
    case 4: hipLaunchKernelGGL((lip_linear_kernel<HS, 4>), grid1, block1, 0, stream, p, q_jobs, x_jobs); break;  \
    default: hipLaunchKernelGGL((lip_linear_kernel<HS, 8>), grid1, block1, 0, stream, p, q_jobs, x_jobs); break; \
    }
    switch (steps) {
    case 4: LIP_LINEAR(2) break;
    case 8: LIP_LINEAR(4) break;
    case 12: LIP_LINEAR(6) break;
    default: return hipErrorInvalidValue;
    }
#undef LIP_LINEAR
    return hipGetLastError();
}

hipError_t lip_launch(const LipParams &p, hipStream_t stream)
{
    hipError_t e = lip_launch_linear(p, stream);
    if (e != hipSuccess) return e;
    return lip_launch_finish(p, stream);
}

hipError_t lip_launch_finish(const LipParams &p, hipStream_t stream)
{
    const int q_wgs = lip_finish_query_wgs(p);
    if (lip_q_on_matrix_cores(p)) {
        // the query rows on the matrix cores, in passes of 32 rows per wave, as many workgroups as are resident at once
        const int npass = (p.T * p.n_heads + 31) / 32;
        const int cus = cu_count();
        if (cus <= 0) return hipErrorNoDevice;
        int wgs = (npass + QFP_WAVES - 1) / QFP_WAVES;
        const int resident = cus * (160 * 1024 / LIP_QFP_LDS);
        wgs = wgs > resident ? resident : wgs;
        hipLaunchKernelGGL(lip_finish_query_prefill_kernel, dim3((unsigned)wgs), dim3(64 * QFP_WAVES), 0, stream, p);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        // key rows and weights: eight tokens per workgroup
        hipLaunchKernelGGL(lip_finish_tokens_prefill_kernel, dim3((unsigned)((p.T + FIN_WAVES - 1) / FIN_WAVES)), dim3(64 * FIN_WAVES), 0, stream, p);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(lip_finish_kernel, dim3((unsigned)(q_wgs + p.T)), dim3(64 * FIN_WAVES), 0, stream, p, q_wgs);
    return hipGetLastError();
}

}  // namespace pto
