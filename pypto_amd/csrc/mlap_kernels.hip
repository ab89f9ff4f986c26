// MLA prolog for gfx950, the variant with bf16 down-projections, an int8 query up-projection and an
// int8 latent cache with four fp32 scales per token: from a decode batch of hidden states it produces
// the absorbed query (nope and rope parts), the int8 normalised query latent with its scale (input of
// the indexer prolog), and writes the new latent / rope / scale rows of the paged caches.
//
// Arithmetic (reference golden: examples/models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py:137-282;
// operator graph: examples/models/deepseek_v32_exp/mla_prolog_quant_impl.py:502-707).  Every fp32 sum
// has a fixed order (all products are bf16 x bf16, exact in fp32): sums over the hidden axis in blocks of
// 64 ascending, eight block sums ascending into a group sum, group sums ascending; the RMS sums as a
// balanced tree over the 128 channels of a slab, slab sums ascending; the 128-term sums against w_uk
// ascending.  In that form only the exact integer projection runs on the matrix cores; the caller may let the
// sums against w_uk, and from MLAP_MFMA_MIN_TOKENS tokens on the sums over the hidden axis, run there as well
// (MlapParams::absorb_exact = 0: the same exact products in the cores' own summation order).
//
// Four launches; below MLAP_MFMA_MIN_TOKENS tokens (decode):
//   mlap_xlinear_kernel  x . [w_dq | w_dkv_kr] (xlinear_fixed.h): one workgroup of eight waves per (slab of 128
//                        columns, group of 512 hidden rows, 8 tokens); each wave takes a 64-row block (staged by
//                        LDS-DMA, hidden states widened to fp32 in LDS), block sums meet in LDS and are
//                        chained into the group sum.
//   mlap_mid_kernel      per token: group sums chained, bf16, RMS norm (one wave per slab), per-token
//                        int8 quantisation of the query latent; RMS norm and per-slab quantisation of
//                        the key latent, rope of the key, scatter into the caches.
//   qproj_kernel         int8 projection of the query latent (shared job code: LDS-DMA tile,
//                        transposing 8-bit LDS reads, v_mfma_i32_32x32x32_i8), partial sums per quarter.
//   mlap_finish_kernel   per (head, half of the 512 output columns, 8 tokens): partial sums added and
//                        de-quantised, rope part rotated and stored, nope part times the head's w_uk
//                        slice (staged in LDS by LDS-DMA): on the matrix cores, or one output column per lane.
// For the fused operator the first and the third of these carry the lightning-indexer prolog's first stage along
// (MlapRider in mlap_kernels.h: its hidden-axis sums have this prolog's fixed order, its projection this one's q_norm).
// From MLAP_MFMA_MIN_TOKENS tokens on (prefill chunks) the stages take forms of their own:
//   mlap_xlinear_mfma_kernel   the sums over the hidden axis on the matrix cores (xlinear_mfma.h) unless the fixed
//                        order is asked for: per workgroup a 128-column slab x 128 tokens x a range of the hidden
//                        axis, v_mfma_f32_32x32x16_bf16 with the row-major weight chunk as the transposed operand.
//                        The launch's first workgroups take the 64 rope columns of w_dkv_kr in their fixed order
//                        instead (the rotated key allows no outlier under the reference's acceptance rule).
//   qproj_prefill_kernel, qproj_prefill256_kernel   the projection unsplit (prolog_common.h), a workgroup per
//                        128 x 128 or 256 x 256 tile over the whole reduction axis; results leave de-quantised.
//   mlap_finish_prefill_kernel   per (head, run of 32-token blocks): the head's whole w_uk staged once
//                        (prolog_finish.h), absorb product on the matrix cores.
#include <cstring>

#include "mlap_kernels.h"
#include "prolog_common.h"
#include "prolog_finish.h"
#include "lip_xjob.h"
#include "xlinear_fixed.h"
#include "xlinear_mfma.h"

#pragma clang fp contract(off)

namespace pto {
namespace {

static_assert(QPROJ_KSPLIT == QPROJ_KSPLIT_HOST, "workspace sizing and kernels disagree");

static_assert(XL_BLOCK == MLAP_XBLOCK && XL_GROUP == MLAP_XGROUP && XL_TOK == MLAP_XTOK, "workspace sizing and kernels disagree");
constexpr int RIDER_XCOLS = 192;     // columns of a row of the rider's group sums: wk's 128, then w_proj's 64

// Fixed-order sums over the hidden axis (xlinear_fixed.h).  Column slabs: 0 .. q_lora/128 - 1 of w_dq, then four
// slabs of w_dkv_kr's latent part and one half slab (64 columns) of its rope part.
// With a rider (mlap_kernels.h) there is one slab more, wk's 128 columns, and the rope slab's upper half is w_proj.
__global__ __launch_bounds__(64 * XL_WAVES) void mlap_xlinear_kernel(const MlapParams p, const int nslabs, const int ngroups, const MlapRider rd)
{
    __shared__ __attribute__((aligned(16))) uint8_t smem[XL_LDS];
    const int slab = blockIdx.x % nslabs;
    const int g = (blockIdx.x / nslabs) % ngroups;
    const int t0 = (blockIdx.x / nslabs / ngroups) * XL_TOK;
    const int qslabs = p.q_lora / 128;
    const int nc = p.q_lora + MLAP_KV + MLAP_ROPE;
    const bool isq = slab < qslabs;
    XlSlab sl;
    if (slab == qslabs + 5) {
        sl.w = reinterpret_cast<const uint8_t *>(rd.wk);
        sl.pitch = 256;
        sl.wbytes = 256;
        sl.out = rd.xpart + (size_t)g * p.T * RIDER_XCOLS;
        sl.out_pitch = RIDER_XCOLS;
    } else {
        sl.w = isq ? reinterpret_cast<const uint8_t *>(p.w_dq) + slab * 256 : reinterpret_cast<const uint8_t *>(p.w_dkvkr) + (slab - qslabs) * 256;
        sl.pitch = (isq ? p.q_lora : MLAP_KV + MLAP_ROPE) * 2;
        sl.wbytes = (!isq && slab - qslabs == 4) ? 128 : 256;
        sl.out = p.xpart + (size_t)g * p.T * nc + slab * 128;
        sl.out_pitch = nc;
        if (sl.wbytes == 128 && rd.w_proj != nullptr) {
            sl.wbytes = 256;
            sl.w_hi = reinterpret_cast<const uint8_t *>(rd.w_proj);
            sl.pitch_hi = 128;
            sl.out_hi = rd.xpart + (size_t)g * p.T * RIDER_XCOLS + 128;
            sl.out_pitch_hi = RIDER_XCOLS;
        }
    }
    xl_body(sl, p.x, p.T, p.h, g, t0, smem);
}

// ---------------------------------------------------------------------------------------------
// Prefill form of the first launch: the same product on the matrix cores (xlinear_mfma.h), for MLAP_MFMA_MIN_TOKENS tokens and more
// when the caller has not asked for the fixed-order sums.  workgroup = (slab of 128 columns of [w_dq | w_dkv_kr],
// one of nsplit ranges of the hidden axis, 128 tokens); the 64 rope columns are a narrow slab of their own.
static_assert(XM_KC == MLAP_XBLOCK, "the workspace is sized in chunks of the hidden axis");

// The first rope_wgs workgroups of the launch (a multiple of eight, so that the XCD-wise order of the others keeps)
// take the 64 rope columns of w_dkv_kr instead, in their fixed order at every size (xlinear_fixed.h, the four-wave DPP
// form; workgroup = (group of eight blocks, 16 tokens)): the reference's acceptance rule allows the rotated key no
// outlier at all (deepseekv32_mla_prolog_quant.py:688: atol 1e-4, rtol 2^-7 per element, ratio 0), and a sum that
// lands next to a bf16 rounding boundary in another order moves a small rotated value by more than that.
// The fused prolog's rider: workgroups past the launch's own run the indexer prolog's fixed-order sums over the
// hidden axis (lip_xjob.h), a wave per job, beside the matrix-core workgroups (two workgroups fit a compute unit).
struct MlapXRider {
    LipParams lip;
    int wgs;        // rider workgroups (0: none)
    int x_jobs;
    int xtok;
};
constexpr int XM_RIDER_LDS = 4 * X_REGION_BYTES;
constexpr int XM_KERNEL_LDS = XM_LDS > XM_RIDER_LDS ? XM_LDS : XM_RIDER_LDS;
static_assert(XR_LDS <= XM_LDS, "the rope jobs fit the launch's LDS");
static_assert(2 * XM_KERNEL_LDS <= 160 * 1024, "two workgroups share a compute unit");
__global__ __launch_bounds__(256) void mlap_xlinear_mfma_kernel(const MlapParams p, const int nslabs, const int nsplit, const int rope_wgs,
                                                                const int rope_groups, const int own_wgs, const MlapXRider rider)
{
    __shared__ __attribute__((aligned(16))) uint8_t smem[XM_KERNEL_LDS];
    if ((int)blockIdx.x >= own_wgs) {
        const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        x_linear_jobs(rider.lip, smem + w * X_REGION_BYTES, ((int)blockIdx.x - own_wgs) * 4 + w, rider.wgs * 4, rider.x_jobs, rider.xtok);
        return;
    }
    if ((int)blockIdx.x < rope_wgs) {
        const int j = blockIdx.x;
        const int g = j % rope_groups;
        const int t0 = (j / rope_groups) * XD_TOK;
        if (t0 >= p.T) return;                         // padding of the count to a multiple of eight
        const int nc = p.q_lora + MLAP_KV + MLAP_ROPE;
        XlSlab sl;
        sl.w = reinterpret_cast<const uint8_t *>(p.w_dkvkr) + MLAP_KV * 2;
        sl.pitch = (MLAP_KV + MLAP_ROPE) * 2;
        sl.wbytes = MLAP_ROPE * 2;
        sl.out = p.xpart + (size_t)g * p.T * nc + p.q_lora + MLAP_KV;
        sl.out_pitch = nc;
        xr_body(sl, p.x, p.T, p.h, g, t0, smem);
        return;
    }
    const int bid = (int)blockIdx.x - rope_wgs;
    // Workgroups go round the eight XCDs, each with an L2 of its own, and the working set (hidden states + weights)
    // is several times one L2: the jobs of a slab (its ranges of h x token tiles) all run on XCD slab % 8, so a slab's
    // weights cross into one L2 only and every XCD reads the hidden states once for its two or so slabs.  The slabs
    // left over when their number is no multiple of eight are dealt out job by job.
    const int per_slab = nsplit * ((p.T + XM_TOK - 1) / XM_TOK);
    const int xcd = bid & 7, j = bid >> 3;
    const int full = nslabs >> 3;
    int slab, rem;
    if (j < full * per_slab) {
        slab = xcd + 8 * (j / per_slab);
        rem = j % per_slab;
    } else {
        const int e = (j - full * per_slab) * 8 + xcd;
        if (e >= (nslabs & 7) * per_slab) return;      // the whole workgroup leaves, before any barrier
        slab = 8 * full + e / per_slab;
        rem = e % per_slab;
    }
    const int sp = rem % nsplit;
    const int t0 = (rem / nsplit) * XM_TOK;
    const int qslabs = p.q_lora / 128;
    const int nc = p.q_lora + MLAP_KV + MLAP_ROPE;
    const bool isq = slab < qslabs;
    XmSlab sl;
    sl.w = isq ? reinterpret_cast<const uint8_t *>(p.w_dq) + slab * 256 : reinterpret_cast<const uint8_t *>(p.w_dkvkr) + (slab - qslabs) * 256;
    sl.pitch = (isq ? p.q_lora : MLAP_KV + MLAP_ROPE) * 2;
    sl.pieces = !isq && slab - qslabs == 4 ? 8 : 16;
    sl.out = p.xpart + (size_t)sp * p.T * nc + slab * 128;
    sl.out_pitch = nc;
    const int nchunks = p.h / XM_KC;
    xm_body(sl, p.x, p.T, p.h, t0, (int)((long long)sp * nchunks / nsplit), (int)((long long)(sp + 1) * nchunks / nsplit), smem);
}

// ---------------------------------------------------------------------------------------------
constexpr int MID_WAVES = MLAP_MAX_QLORA / 128;   // 12

// sum over the wave's 128 values of rn(rn(v*v) * coef) as a balanced tree over neighbours
__device__ __forceinline__ float slab_square_sum(const float v0, const float v1, const float coef)
{
    return pair_tree_sum(__fmul_rn(__fmul_rn(v0, v0), coef), __fmul_rn(__fmul_rn(v1, v1), coef));
}

// Workgroup 2t: the query latent of token t (one wave per slab of 128 channels).  Workgroup 2t+1: its
// key latent (waves 0..3) and key rope part (wave 4).
// ngroups partial sums over the hidden axis per column, ngroups_rope for the 64 rope columns (which keep the fixed-order
// form's groups when the other columns come from the matrix cores).
__global__ __launch_bounds__(64 * MID_WAVES) void mlap_mid_kernel(const MlapParams p, const int ngroups_other, const int ngroups_rope)
{
    __shared__ float slabsum[MID_WAVES];
    __shared__ float slabmax[MID_WAVES];
    const int l = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = blockIdx.x >> 1;
    const bool kvtype = blockIdx.x & 1;
    const int qslabs = p.q_lora / 128;
    const int nc = p.q_lora + MLAP_KV + MLAP_ROPE;
    const int nslab = kvtype ? 4 : qslabs;                               // slabs under the norm
    const bool rope_wave = kvtype && w == 4;
    const bool active = w < nslab || rope_wave;
    const int ngroups = rope_wave ? ngroups_rope : ngroups_other;
    const int col = (kvtype ? p.q_lora : 0) + w * 128 + 2 * (rope_wave ? (l & 31) : l);

    // Everything the chain below needs from memory is requested before the first value is looked at: the
    // cache row, the norm weights, the rotation factors and the group sums, sixteen groups at a time
    // (taken one after the other, the fourteen group loads of a 7168-wide hidden axis alone were fourteen
    // memory latencies).
    const long long dst = kvtype ? p.cache_index[t] : -1;
    uint32_t gm = 0;
    if (w < nslab) gm = reinterpret_cast<const uint32_t *>(kvtype ? p.gamma_ckv : p.gamma_cq)[w * 64 + l];
    uint16_t cs0 = 0, cs1 = 0, sn0 = 0, sn1 = 0;
    if (rope_wave && l < 32) {
        cs0 = p.cos[(size_t)t * MLAP_ROPE + l];
        cs1 = p.cos[(size_t)t * MLAP_ROPE + 32 + l];
        sn0 = p.sin[(size_t)t * MLAP_ROPE + l];
        sn1 = p.sin[(size_t)t * MLAP_ROPE + 32 + l];
    }
    float v0 = 0.f, v1 = 0.f;
    if (active) {
        const float *src = p.xpart + (size_t)t * nc + col;
        for (int g0 = 0; g0 < ngroups; g0 += 16) {
            f32x2 v[16];
#pragma unroll
            for (int g = 0; g < 16; ++g)
                v[g] = *reinterpret_cast<const f32x2 *>(src + (size_t)(g0 + g < ngroups ? g0 + g : ngroups - 1) * p.T * nc);
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                if (g0 + g < ngroups) {
                    v0 = __fadd_rn(v0, v[g][0]);
                    v1 = __fadd_rn(v1, v[g][1]);
                }
            }
        }
        v0 = bf16_round_f32(v0);
        v1 = bf16_round_f32(v1);
    }
    const bool dst_ok = dst >= 0 && dst < p.cache_rows;

    if (rope_wave) {
        // lane l < 32 holds channels 2l and 2l+1, which after the de-interleave are channels l and 32+l:
        // the two partners of one rotation
        if (l < 32) {
            const float c0 = bf16_bits_to_f32(cs0), c1 = bf16_bits_to_f32(cs1);
            const float s0 = bf16_bits_to_f32(sn0), s1 = bf16_bits_to_f32(sn1);
            const float r0 = __builtin_fmaf(v0, c0, (-v1) * s0);      // products exact: one rounding
            const float r1 = __builtin_fmaf(v1, c1, v0 * s1);
            if (dst_ok) {
                p.kr_cache[(size_t)dst * MLAP_ROPE + l] = (uint16_t)(pack_bf16x2(r0, 0.f) & 0xffffu);
                p.kr_cache[(size_t)dst * MLAP_ROPE + 32 + l] = (uint16_t)(pack_bf16x2(r1, 0.f) & 0xffffu);
            }
        }
    }
    const int n = kvtype ? MLAP_KV : p.q_lora;
    if (w < nslab) {
        const float ss = slab_square_sum(v0, v1, (float)(1.0 / (double)n));
        if (l == 0) slabsum[w] = ss;
    }
    __syncthreads();
    float y0 = 0.f, y1 = 0.f;
    if (w < nslab) {
        float s = 0.f;
        for (int j = 0; j < nslab; ++j) s = __fadd_rn(s, slabsum[j]);
        const float d = __builtin_sqrtf(__fadd_rn(s, kvtype ? p.eps_ckv : p.eps_cq));   // correctly rounded (__fsqrt_rn is the 1-ulp hardware root here)
        y0 = bf16_round_f32(__fmul_rn(__fdiv_rn(v0, d), __uint_as_float(gm << 16)));
        y1 = bf16_round_f32(__fmul_rn(__fdiv_rn(v1, d), __uint_as_float(gm & 0xffff0000u)));
        const float m = wave_max_f32(fmaxf(fabsf(y0), fabsf(y1)));
        if (l == 0) slabmax[w] = m;
    }
    __syncthreads();
    if (w < nslab) {
        float amax = slabmax[w];
        if (!kvtype)
            for (int j = 0; j < nslab; ++j) amax = fmaxf(amax, slabmax[j]);
        float deq;
        const uint16_t q = quant_pair_amax(y0, y1, amax, deq);
        if (!kvtype) {
            reinterpret_cast<uint16_t *>(p.q_norm + (size_t)t * p.q_lora)[w * 64 + l] = q;
            if (w == 0 && l == 0) p.q_norm_scale[t] = deq;
        } else if (dst_ok) {
            reinterpret_cast<uint16_t *>(p.kv_cache + (size_t)dst * MLAP_KV)[w * 64 + l] = q;
            if (l == 0) p.k_scale_cache[(size_t)dst * 4 + w] = deq;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// One workgroup (two waves, one half of a quarter tile each) walks the jobs blockIdx.x, + gridDim.x, ...:
// the tile of the next job is requested into the other buffer before the current one is consumed, so the
// weights stream without a gap between jobs.  The wave pair adds its accumulators through one of two
// parking areas, alternating, with one barrier per job.
template <int HS>
constexpr int qproj_lds_bytes()
{
    return 4 * HS * (32 * 128 + 1024) + 2 * LIN_RED_BYTES;
}

// Jobs [0, njobs_a) belong to projection pa, jobs [njobs_a, njobs) to pb (same q_norm and reduction axis: the rider's).
template <int HS>
__global__ __launch_bounds__(128) void qproj_kernel(const QProj pa, const int njobs_a, const QProj pb, const int njobs)
{
    constexpr int BUF = HS * (32 * 128 + 1024);
    constexpr int NREQ = HS * 5;                       // requests of one job per wave
    __shared__ __attribute__((aligned(16))) uint8_t smem[qproj_lds_bytes<HS>()];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = threadIdx.x & 63;
    uint8_t *bufs = smem + w * 2 * BUF;
    uint8_t *park = smem + 4 * BUF;
    int job = blockIdx.x;
    const auto issue = [&](uint8_t *region, const int j) {
        if (j < njobs_a) q_issue<HS>(pa, region, j, w);
        else q_issue<HS>(pb, region, j - njobs_a, w);
    };
    if (job < njobs) issue(bufs, job);
    for (int k = 0; job < njobs; job += gridDim.x, ++k) {
        const int next = job + gridDim.x;
        if (next < njobs) {
            issue(bufs + ((k + 1) & 1) * BUF, next);
            VM_WAIT(NREQ);
        } else {
            VM_WAIT(0);
        }
        i32x16 acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][r] = 0;
        const uint8_t *region = bufs + (k & 1) * BUF;
#pragma unroll
        for (int s = 0; s < HS; ++s) q_step<HS>(region, s, l, acc);
        uint8_t *pk = park + (k & 1) * LIN_RED_BYTES;
        if (w == 1) q_pair_park(pk, l, acc);
        __syncthreads();
        if (w == 0) {
            if (job < njobs_a) q_pair_store_from(pa, pk, job, l, acc);
            else q_pair_store_from(pb, pk, job - njobs_a, l, acc);
        }
    }
}

// TB: token blocks per tile (prolog_common.h).  HS > 0: workgroups past the launch's own run the fused prolog's
// rider, the indexer prolog's split int8 projection (one job of a wave pair each, HS steps of 32 rows per half; the
// other two waves only keep the barrier company), beside the tiles' workgroups (two workgroups fit a compute unit).
template <int TB, int HS>
__global__ __launch_bounds__(256) void qproj_prefill_kernel(const QProj p, const int njobs, const QProj rider)
{
    constexpr int RIDER_LDS = HS > 0 ? 2 * lin_region_bytes<(HS > 0 ? HS : 1)>() : 0;
    constexpr int LDS = QPF_LDS > RIDER_LDS ? QPF_LDS : RIDER_LDS;
    static_assert(2 * LDS <= 160 * 1024, "two workgroups share a compute unit");
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS];
    if (HS > 0 && (int)blockIdx.x >= njobs) {
        constexpr int H = HS > 0 ? HS : 1;
        const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = threadIdx.x & 63;
        const int job = (int)blockIdx.x - njobs;
        i32x16 acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][r] = 0;
        uint8_t *region = lds + (w & 1) * lin_region_bytes<H>();
        if (w < 2) {
            q_half_job<H>(rider, region, job, w, acc);
            if (w == 1) q_pair_park(region, l, acc);
        }
        __syncthreads();
        if (w == 0) q_pair_store<H>(rider, lds, job, l, acc);
        return;
    }
    q_prefill_body<TB>(p, q_prefill_job_of((int)blockIdx.x, njobs), lds);
}

__global__ __launch_bounds__(512) void qproj_prefill256_kernel(const QProj p, const int njobs)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[QP2_LDS];
    q_prefill256_body(p, q_prefill_job_of((int)blockIdx.x, njobs), lds);
}

// ---------------------------------------------------------------------------------------------
// Last launch: prolog_finish.h.
__global__ __launch_bounds__(256) void mlap_finish_kernel(const MlapParams p)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[MLAP_FIN_LDS];
    mlap_finish_body(p, (int)blockIdx.x, lds);
}

__global__ __launch_bounds__(64 * FINP_WAVES) void mlap_finish_prefill_kernel(const MlapParams p, const int per)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[MLAP_FINP_LDS];
    mlap_finish_prefill_body(p, (int)blockIdx.x, per, lds);
}

}  // namespace

bool mlap_finish_is_prefill(const MlapParams &p) { return mlap_prefill_forms(p); }

void mlap_finish_prefill_shape(const MlapParams &p, int &per, int &wgs)
{
    // runs of up to 16 blocks of 32 tokens per workgroup, two runs at least so that 128 heads fill the chip
    const int nblocks = (p.T + FINP_TOK - 1) / FINP_TOK;
    per = (nblocks + 1) / 2;
    per = per > 16 ? 16 : per;
    wgs = p.n_heads * ((nblocks + per - 1) / per);
}

hipError_t mlap_launch_finish(const MlapParams &p, hipStream_t stream)
{
    if (mlap_finish_is_prefill(p)) {
        int per, wgs;
        mlap_finish_prefill_shape(p, per, wgs);
        hipLaunchKernelGGL(mlap_finish_prefill_kernel, dim3((unsigned)wgs), dim3(64 * FINP_WAVES), 0, stream, p, per);
    } else {
        hipLaunchKernelGGL(mlap_finish_kernel, dim3((unsigned)mlap_finish_wgs(p)), dim3(256), 0, stream, p);
    }
    return hipGetLastError();
}

int mlap_finish_wgs(const MlapParams &p) { return p.n_heads * 2 * ((p.T + MLAP_XTOK - 1) / MLAP_XTOK); }

hipError_t mlap_launch_front(const MlapParams &p, hipStream_t stream, const MlapRider *rider, const LipParams *lip_rider)
{
    const int nblk = p.h / MLAP_XBLOCK;
    int ngroups = (nblk + MLAP_XGROUP - 1) / MLAP_XGROUP;
    const int ngroups_fixed = ngroups;
    const int nslabs = p.q_lora / 128 + 5;
    if (rider != nullptr && !mlap_takes_rider(p)) return hipErrorInvalidValue;
    if (lip_rider != nullptr && !mlap_takes_lip_rider(p)) return hipErrorInvalidValue;
    const MlapRider rd = rider != nullptr ? *rider : MlapRider{nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    if (mlap_prefill_forms(p)) {
        // prefill sizes: the sums over the hidden axis on the matrix cores, in as many ranges of the hidden axis
        // (partial sums per token) as give about two workgroups per compute unit, MLAP_XM_MAX_SPLITS at most
        const int nchunks = p.h / XM_KC;
        const int ttiles = (p.T + XM_TOK - 1) / XM_TOK;
        const int cus = cu_count();
        if (cus <= 0) return hipErrorNoDevice;
        ngroups = 2 * cus / (nslabs * ttiles);
        ngroups = ngroups < 1 ? 1 : ngroups;
        ngroups = ngroups > MLAP_XM_MAX_SPLITS ? MLAP_XM_MAX_SPLITS : ngroups;
        ngroups = ngroups > nchunks ? nchunks : ngroups;
        // every slab but the last, the rope columns, which keep their fixed-order sums
        const int mslabs = nslabs - 1;
        const int per_slab = ngroups * ttiles;
        const int wgs = 8 * ((mslabs >> 3) * per_slab + ((mslabs & 7) * per_slab + 7) / 8);   // the kernel's XCD-wise job order
        const int rope_wgs = (ngroups_fixed * ((p.T + XD_TOK - 1) / XD_TOK) + 7) / 8 * 8;
        MlapXRider xr;
        xr.wgs = 0;
        xr.x_jobs = xr.xtok = 0;
        if (lip_rider != nullptr) {
            xr.lip = *lip_rider;
            xr.xtok = lip_xtok(lip_rider->T);
            xr.x_jobs = lip_x_jobs(*lip_rider, xr.xtok);
            xr.wgs = (xr.x_jobs + 3) / 4;
            xr.wgs = xr.wgs > 2 * cus ? 2 * cus : xr.wgs;
        } else {
            std::memset(&xr.lip, 0, sizeof xr.lip);
        }
        hipLaunchKernelGGL(mlap_xlinear_mfma_kernel, dim3((unsigned)(rope_wgs + wgs + xr.wgs)), dim3(256), 0, stream, p, mslabs, ngroups, rope_wgs,
                           ngroups_fixed, rope_wgs + wgs, xr);
    } else {
        const int tgroups = (p.T + MLAP_XTOK - 1) / MLAP_XTOK;
        const int xslabs = nslabs + (rider != nullptr ? 1 : 0);
        hipLaunchKernelGGL(mlap_xlinear_kernel, dim3((unsigned)(xslabs * ngroups * tgroups)), dim3(64 * XL_WAVES), 0, stream, p, xslabs, ngroups, rd);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(mlap_mid_kernel, dim3((unsigned)(2 * p.T)), dim3(64 * MID_WAVES), 0, stream, p, ngroups, ngroups_fixed);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    const QProj qp = {p.q_norm, p.w_uqqr, p.qpart, p.T, p.q_lora, p.n_heads * MLAP_QHEAD / 128, p.q_norm_scale, p.w_qb_scale};
    if (mlap_qsplits(p) == 1) {
        if (p.q_lora % (32 * QPF_STEPS)) return hipErrorInvalidValue;
        const int cus = cu_count();
        if (cus <= 0) return hipErrorNoDevice;
        const int njobs256 = q_prefill256_jobs(qp);
        if (4 * njobs256 >= 3 * cus) {                 // enough 256 x 256 tiles to fill the chip
            hipLaunchKernelGGL(qproj_prefill256_kernel, dim3((unsigned)njobs256), dim3(512), 0, stream, qp, njobs256);
            return hipGetLastError();
        }
        const int njobs = q_prefill_jobs(qp);
        const dim3 g((unsigned)njobs), b(256);
        const int tbk = q_prefill_token_blocks(p.T);
        if (lip_rider != nullptr) {
            // the indexer prolog's split projection rides along: one more workgroup per job of a wave pair
            const LipParams &lp = *lip_rider;
            const QProj qr = {lp.q_norm, lp.w_qb, lp.qpart, lp.T, lp.q_lora, lp.n_heads, lp.q_norm_scale, lp.w_qb_scale};
            const int rjobs = lp.n_heads * QPROJ_KSPLIT * ((lp.T + 31) / 32);
            const dim3 gr((unsigned)(njobs + rjobs));
            const int steps = lp.q_lora / QPROJ_KSPLIT / 32;
#define QPF_RIDER(TBV)                                                                                       \
    switch (steps) {                                                                                         \
    case 4: hipLaunchKernelGGL((qproj_prefill_kernel<TBV, 2>), gr, b, 0, stream, qp, njobs, qr); break;     \
    case 8: hipLaunchKernelGGL((qproj_prefill_kernel<TBV, 4>), gr, b, 0, stream, qp, njobs, qr); break;     \
    case 12: hipLaunchKernelGGL((qproj_prefill_kernel<TBV, 6>), gr, b, 0, stream, qp, njobs, qr); break;    \
    default: return hipErrorInvalidValue;                                                                    \
    }
            if (tbk == 1) { QPF_RIDER(1) } else { QPF_RIDER(2) }
#undef QPF_RIDER
            return hipGetLastError();
        }
        switch (tbk) {
        case 1: hipLaunchKernelGGL((qproj_prefill_kernel<1, 0>), g, b, 0, stream, qp, njobs, qp); break;
        case 2: hipLaunchKernelGGL((qproj_prefill_kernel<2, 0>), g, b, 0, stream, qp, njobs, qp); break;
        default: hipLaunchKernelGGL((qproj_prefill_kernel<4, 0>), g, b, 0, stream, qp, njobs, qp);
        }
        return hipGetLastError();
    }
    const int qjobs_a = qp.nslabs * QPROJ_KSPLIT * ((p.T + 31) / 32);
    const QProj qr = {p.q_norm, rd.w_qb, rd.qpart, p.T, p.q_lora, rd.q_slabs, p.q_norm_scale, nullptr};
    const int qjobs = qjobs_a + qr.nslabs * QPROJ_KSPLIT * ((p.T + 31) / 32);
    // as many workgroups as fit at once (by their LDS), every one with the same number of jobs where possible
    const int steps = p.q_lora / QPROJ_KSPLIT / 32;
    const int lds = steps == 12 ? qproj_lds_bytes<6>() : (steps == 8 ? qproj_lds_bytes<4>() : qproj_lds_bytes<2>());
    const int cus = cu_count();
    if (cus <= 0) return hipErrorNoDevice;
    const int slots = cus * (160 * 1024 / lds);
    const int rounds = (qjobs + slots - 1) / slots;
    const dim3 qgrid((unsigned)((qjobs + rounds - 1) / rounds));
    switch (steps) {
    case 4: hipLaunchKernelGGL(qproj_kernel<2>, qgrid, dim3(128), 0, stream, qp, qjobs_a, qr, qjobs); break;
    case 8: hipLaunchKernelGGL(qproj_kernel<4>, qgrid, dim3(128), 0, stream, qp, qjobs_a, qr, qjobs); break;
    case 12: hipLaunchKernelGGL(qproj_kernel<6>, qgrid, dim3(128), 0, stream, qp, qjobs_a, qr, qjobs); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t mlap_launch(const MlapParams &p, hipStream_t stream)
{
    hipError_t e = mlap_launch_front(p, stream);
    if (e != hipSuccess) return e;
    return mlap_launch_finish(p, stream);
}

}  // namespace pto
