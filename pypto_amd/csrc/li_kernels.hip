// Lightning indexer (decode), gfx950 (MI355X): key scoring and top-k select.
//
// Semantics: lightning_indexer_decode_compute of the reference example
// (examples/models/deepseek_v32_exp/lightning_indexer_quant_impl.py:138-312), golden
// deepseekv32_lightning_indexer_quant.py:184-269:
//   x[h, j]  = fp16_rne(relu(q[h,:] . k[j,:]) / 2048)                int8 dot, exact in int32
//   score[j] = (sum_h w_scale[h] * x[h, j]) * k_scale[j]             fp32
// with the two orders the golden leaves to its libraries fixed as: head sum h ascending with the
// product rounded before the add (no fused multiply-add); select order (score descending, position
// ascending), -0.0 == +0.0.
//
// Kernels
//   li_score_kernel   w_scale[h] = fp16(q_scale * weight) if both fp16, else the fp32 product;
//                     one wave per run of 64-key pairs of blocks: the key rows travel from the paged
//                     cache into the wave's own LDS buffers by LDS-DMA (whole cache lines, two pairs
//                     ahead), v_mfma_i32_32x32x32_i8 with A = the token's 64 query heads (two 32-row
//                     operands resident in registers) and B = 32 key rows read from LDS in operand
//                     layout; a half-wave swap gives every lane all 64 heads of one key, summed in
//                     registers with the per-head factors in scalar registers; scores to a
//                     [T, max_seq] fp32 workspace, and one score of every 16 positions to a compact
//                     sample array behind it
//   li_select_kernel  one workgroup per query token, keys ordered by the strict word
//                     (score image << 32 | ~position): a histogram of up to 4096 sampled scores (the
//                     compact array the score kernel left) gives a pivot, one pass over the row
//                     compacts the keys above it, those are spread over 2048 buckets linear in the
//                     score and ordered inside buckets by counting; select_streaming (radix select
//                     over the row in memory + bitonic sort) is the capacity-free form it falls back to
#include <type_traits>

#include "common.h"
#include "li_kernels.h"
#include "pypto_amd_sfa.h"

// The head sum is defined as a rounded multiply followed by a rounded add.  __fmul_rn/__fadd_rn are
// plain operators to the compiler, so contraction is switched off for this whole file.  The pragma
// is honoured only when the file is compiled with -ffp-contract=on or off: hipcc's default, "fast",
// lets the backend fuse regardless.
#pragma clang fp contract(off)

namespace pto {
namespace {


__device__ __forceinline__ float load_scalar(const void *p, size_t i, int dt)
{
    if (dt == PTO_DT_FP32) return static_cast<const float *>(p)[i];
    const uint16_t h = static_cast<const uint16_t *>(p)[i];
    if (dt == PTO_DT_BF16) return bf16_bits_to_f32(h);
    return (float)__builtin_bit_cast(_Float16, h);
}

// w_scale[h] = fp16(q_scale * weight) when both are fp16 (one fp16 rounding of the exact product),
// else the fp32 product
__device__ __forceinline__ float w_scale_of(const LiParams &p, const size_t i)
{
    const float qs = load_scalar(p.q_scale, i, p.q_dt);
    const float wt = load_scalar(p.weight, i, p.w_dt);
    float prod = __fmul_rn(qs, wt);
    if (p.q_dt == PTO_DT_FP16 && p.w_dt == PTO_DT_FP16) prod = (float)(_Float16)prod;
    return prod;
}

// order-preserving image of a score: larger score <=> larger key; -0.0 and +0.0 map to one key
__device__ __forceinline__ uint32_t score_key(const float x)
{
    uint32_t u = __float_as_uint(x);
    u = u == 0x80000000u ? 0u : u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Wave-wide scan and reductions on DPP (no LDS traffic).  row_shr:n moves a value n lanes up inside
// its row of 16, row_bcast15/31 carry the last lane of a row / of the lower half-wave upward; lanes
// without a source keep the identity passed as the old value.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_u32(const uint32_t identity, const uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)identity, (int)v, CTRL, ROW_MASK, 0xf, false);
}

// inclusive prefix sum over the 64 lanes
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v)
{
    v += dpp_u32<0x111, 0xf>(0u, v);
    v += dpp_u32<0x112, 0xf>(0u, v);
    v += dpp_u32<0x114, 0xf>(0u, v);
    v += dpp_u32<0x118, 0xf>(0u, v);
    v += dpp_u32<0x142, 0xa>(0u, v);
    v += dpp_u32<0x143, 0xc>(0u, v);
    return v;
}

template <typename Op>
__device__ __forceinline__ uint32_t wave_reduce_bits(uint32_t v, const uint32_t identity, Op op)
{
    v = op(v, dpp_u32<0x111, 0xf>(identity, v));
    v = op(v, dpp_u32<0x112, 0xf>(identity, v));
    v = op(v, dpp_u32<0x114, 0xf>(identity, v));
    v = op(v, dpp_u32<0x118, 0xf>(identity, v));
    v = op(v, dpp_u32<0x142, 0xa>(identity, v));
    v = op(v, dpp_u32<0x143, 0xc>(identity, v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);     // lane 63 holds the reduction of all lanes
}

__device__ __forceinline__ float wave_min(const float x)
{
    return __uint_as_float(wave_reduce_bits(__float_as_uint(x), 0x7f800000u, [](uint32_t a, uint32_t b) {
        return __float_as_uint(fminf(__uint_as_float(a), __uint_as_float(b)));
    }));
}

__device__ __forceinline__ float wave_max(const float x)
{
    return __uint_as_float(wave_reduce_bits(__float_as_uint(x), 0xff800000u, [](uint32_t a, uint32_t b) {
        return __float_as_uint(fmaxf(__uint_as_float(a), __uint_as_float(b)));
    }));
}

__device__ __forceinline__ uint32_t wave_max_u32(const uint32_t x)
{
    return wave_reduce_bits(x, 0u, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
}

// fp32 product of one half of a packed fp16 pair with a wave-uniform fp32 factor, rounded once:
// v_fma_mix_f32 widens the fp16 operand on the fly.  The addend +0 turns a product of -0 into +0, which
// no later step can tell apart: the running sum starts at +0 and so never is -0 itself.
template <int HI>
__device__ __forceinline__ float mul_f16_f32(const uint32_t packed, const float w)
{
    float r;
    if (HI)
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "s"(w));
    else
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "s"(w));
    return r;
}

// the same with the factor in a vector register (read from LDS)
template <int HI>
__device__ __forceinline__ float mul_f16_f32_v(const uint32_t packed, const float w)
{
    float r;
    if (HI)
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(w));
    else
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(w));
    return r;
}

// x = fp16(relu(dot) / 2048) for two dots, packed.  v_fma_mixlo/mixhi_f16 scale in fp32 (exact: a power
// of two) and round once to fp16; -|dot|/2048 rounds to a negative fp16 that the packed integer max
// then clears, which equals clearing first.  scale = 2^-11 in a scalar register.
__device__ __forceinline__ uint32_t relu_fp16_pair(const int d0, const int d1, const float scale)
{
    uint32_t packed;
    asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(packed) : "v"((float)d0), "s"(scale));
    asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(packed) : "v"((float)d1), "s"(scale));
    // relu on the bit patterns: a negative fp16 (and -0) is a negative 16-bit integer
    typedef __attribute__((ext_vector_type(2))) short s16x2;
    const s16x2 zero = {0, 0};
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s16x2, packed), zero));
}

// fp16(dot / 2048) for two dots, packed, sign kept
__device__ __forceinline__ uint32_t fp16_pair(const int d0, const int d1, const float scale)
{
    uint32_t packed;
    asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(packed) : "v"((float)d0), "s"(scale));
    asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(packed) : "v"((float)d1), "s"(scale));
    return packed;
}

// two heads of one key: ((x * q_scale) * k_scale, ReLU) * weight, every product rounded to fp16
__device__ __forceinline__ uint32_t dequant_relu_weight(const uint32_t x, const uint32_t qs, const uint32_t ks, const uint32_t w)
{
    typedef __attribute__((ext_vector_type(2))) short s16x2;
    f16x2 v = __builtin_bit_cast(f16x2, x) * __builtin_bit_cast(f16x2, qs);
    v = v * __builtin_bit_cast(f16x2, ks);
    const s16x2 zero = {0, 0};
    v = __builtin_bit_cast(f16x2, __builtin_elementwise_max(__builtin_bit_cast(s16x2, v), zero));
    return __builtin_bit_cast(uint32_t, v * __builtin_bit_cast(f16x2, w));
}

// Sample for the select: of every 16 consecutive positions that all lie inside the sequence, the score
// of one (picked by a hash of the group number) is also written to a compact array, so that the select
// kernel finds a sample of the row in a few contiguous cache lines instead of thousands of scattered ones.
__device__ __forceinline__ bool sample_lane(const int pos, const int cur)
{
    const uint32_t g = (uint32_t)pos >> 4;
    return (uint32_t)(pos & 15) == ((g * 2654435761u) >> 28) && (int)(16u * g + 15u) < cur;
}

constexpr int SC_PAIR_BYTES = 64 * LI_DIM;     // key rows of one staged pair of 32-key blocks
constexpr int SC_BUF_BYTES = SC_PAIR_BYTES + 256;   // + the 64 key scales (one dword per lane)

// One wave scores runs of 64 consecutive keys: two 32-key blocks X and Y per trip.
//   stage  key rows travel from the paged cache into the wave's own LDS buffers with
//          global_load_lds: consecutive lanes fetch consecutive 16-byte chunks, so every request is a
//          run of whole cache lines (loading the operand layout directly touches 32 lines with 32
//          bytes each per instruction and is bound by the address unit).  Chunk c of row r lands at
//          position c ^ (r & 7) of the row, which makes the operand reads below conflict-free.  The
//          pair after the current one is in flight while the current one is scored.
//   MFMA   A = the token's 64 query heads as two 32-row operands (resident in registers), B = 32 key
//          rows read from LDS in operand layout; four accumulators per trip.  With the head
//          permutation below, lane (j, half) of block X's accumulators holds heads 32*half ..
//          32*half + 31 of key X_j, likewise for Y.
//   swap   after relu / scale / fp16 packing, v_permlane32_swap exchanges the upper half-wave of X's
//          registers with the lower half-wave of Y's: lane j < 32 then holds all 64 heads of key X_j
//          and lane 32 + j all 64 heads of key Y_j, the same head in the same register on every lane.
//   sum    every lane runs the sequential head sum h = 0..63 of its own key; the per-head factors are
//          wave-uniform and sit in scalar registers.
// At least two waves per SIMD: the 256 registers that leaves per lane are all architectural, so the
// matrix instructions accumulate in ordinary vector registers and the epilogue reads them directly.
// KDT = dtype code of the key scales: a compile-time choice keeps the scale load free of branches, so
// it stays in flight beside the staged rows.
// VAR = 1: the arithmetic of the reference's chained C++ operator (LightningIndexerTopkImpl,
// framework/src/operator/models/deepseek_v3.2_exp/lightning_indexer.cpp:149-197): fp16(dot/2048) is
// multiplied in fp16 by the head's query scale and by the key's scale before the ReLU, then in fp16 by
// the head's weight; the fp32 head sum (h ascending) is the score.  All three tensors are fp16 then.
// NT = query tokens of one sequence a wave scores per key pass (1 or 2): the reference scores all s1 tokens of
// a batch against a page in one matrix product (lightning_indexer_quant_impl.py:163-169, [S1*64, 128]); here
// a "unit" is a pair of consecutive tokens of a sequence (the last unit of an odd s1 holds one), every staged
// key row and scale serves both, and their per-head factors sit in LDS instead of scalar registers.
template <int KDT, int VAR = 0, int NT = 1>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void li_score_kernel(const LiParams p)
{
    __shared__ __attribute__((aligned(16))) int8_t kstage[4][2][SC_BUF_BYTES];
    __shared__ __attribute__((aligned(16))) float wsc_lds[NT > 1 ? 4 : 1][NT][LI_HEADS];
    const int upb = (p.S1 + NT - 1) / NT;            // units per sequence
    const int nunits = p.B * upb;
    const int w = threadIdx.x >> 6;
    const int l = threadIdx.x & 63;
    const int j = l & 31;
    const int half = l >> 5;
    const int cap = p.maxblk * p.bs;
    int t, key0, ppw;
    if (p.balanced) {
        // Balanced mapping (at most 512 query tokens): the launch has a fixed number of waves; every wave
        // reads all sequence lengths, sizes the runs so that the runs of all tokens just fill the
        // launch, and takes the gw-th run in token order.  Short and long sequences then cost the same
        // number of trips per wave and the whole pass is one round of resident waves.
        const int gw = blockIdx.x * 4 + w;
        const int nwaves = gridDim.x * 4;
        int pairs[8], total = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int tt = l + 64 * i;
            int c = tt < nunits ? p.act[tt / upb] : 0;
            c = c < 0 ? 0 : (c > cap ? cap : c);
            pairs[i] = (c + 63) >> 6;
            total += pairs[i];
        }
        total = (int)wave_incl_scan((uint32_t)total);
        total = __builtin_amdgcn_readlane(total, 63);
        // every token may waste one run on rounding: plan for nwaves - T runs
        ppw = (total + (nwaves - nunits) - 1) / (nwaves - nunits);
        ppw = ppw < 1 ? 1 : (ppw > LI_MAX_PAIRS_PER_WAVE ? LI_MAX_PAIRS_PER_WAVE : ppw);
        int base = 0;                     // runs of all tokens before row i of the token table
        int found = -1;                   // token of this wave's run << 16 | run index... kept separately below
        int found_run = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int runs = (pairs[i] + ppw - 1) / ppw;
            const int incl = (int)wave_incl_scan((uint32_t)runs);
            const int start = base + incl - runs;
            if (gw >= start && gw < start + runs) { found = l + 64 * i; found_run = gw - start; }
            base += __builtin_amdgcn_readlane(incl, 63);
        }
        const unsigned long long hit = __ballot(found >= 0);
        if (hit == 0ull) return;          // more waves than runs
        const int src = __ffsll((long long)hit) - 1;
        t = __builtin_amdgcn_readlane(found, src);
        key0 = __builtin_amdgcn_readlane(found_run, src) * (ppw * 64);
    } else {
        t = blockIdx.y;
        ppw = p.ppw;
        key0 = (blockIdx.x * 4 + w) * (ppw * 64);
    }
    // t is the unit's number up to here; from here on its first token
    const int b = t / upb;
    const int s_first = (t - b * upb) * NT;
    const int nt = p.S1 - s_first < NT ? p.S1 - s_first : NT;     // tokens of this unit (uniform)
    t = b * p.S1 + s_first;
    int cur = p.act[b];
    cur = cur < 0 ? 0 : (cur > cap ? cap : cur);
    if (key0 >= cur) return;
    int npair = (cur - key0 + 63) >> 6;
    npair = npair > ppw ? ppw : npair;
    const int last_blk = ((cur + 31) >> 5) - 1;                  // last 32-key block holding a valid key

    // First cache row of every 32-key block of this wave's run, looked up once: lane i holds the row of
    // block i of the run (32 consecutive positions never straddle a page; a run has at most 64 blocks;
    // blocks past the end of the sequence repeat the last valid block).
    int run_row;
    {
        int blk = (key0 >> 5) + l;
        blk = blk > last_blk ? last_blk : blk;
        const int pos0 = 32 * blk;
        const int page = pos0 / p.bs;
        int pb = p.bt[(size_t)b * p.maxblk + page];
        pb = pb < 0 ? 0 : (pb >= p.nblocks ? p.nblocks - 1 : pb);
        run_row = pb * p.bs + (pos0 - page * p.bs);
    }
    // Requests pair pr into buffer buf: per block four instructions of eight rows each.  Lane l owns
    // LDS slot l of an instruction's 1 KiB, i.e. row l/8 and position l%8, and fetches chunk
    // (l%8) ^ (l/8) of that row; the instruction offset moves the cache address and the LDS address
    // alike.  A ninth instruction stages the dword holding the scale of the key whose sum this lane
    // will hold (X_j on the lower half-wave, Y_j on the upper).  Every load of the loop is written as
    // assembly: the compiler then tracks none of them, and the explicit waits of the trips decide
    // alone how long requests stay outstanding (two pairs ahead).
    const uint32_t lane_off = (uint32_t)((l >> 3) * LI_DIM + (((l & 7) ^ (l >> 3)) << 4));
    const uint32_t lds_base = (uint32_t)__builtin_amdgcn_readfirstlane(
        (int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t *)&kstage[w][0][0]);
    constexpr int KSZ = KDT == PTO_DT_FP32 ? 4 : 2;
    auto request_pair = [&](const int pr, const int buf) {
        const int rx = __builtin_amdgcn_readlane(run_row, 2 * pr), ry = __builtin_amdgcn_readlane(run_row, 2 * pr + 1);
        const int8_t *gx = p.kcache + (size_t)rx * LI_DIM;
        const int8_t *gy = p.kcache + (size_t)ry * LI_DIM;
        const uint32_t dst = lds_base + (uint32_t)(buf * SC_BUF_BYTES);
        asm volatile("s_mov_b32 m0, %2\n\t"
                     "s_nop 0\n\t"
                     "global_load_lds_dwordx4 %0, %1\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:2048\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:3072"
                     :: "v"(lane_off), "s"(gx), "s"(dst) : "memory", "m0");
        asm volatile("s_mov_b32 m0, %2\n\t"
                     "s_nop 0\n\t"
                     "global_load_lds_dwordx4 %0, %1\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:2048\n\t"
                     "global_load_lds_dwordx4 %0, %1 offset:3072"
                     :: "v"(lane_off), "s"(gy), "s"(dst + 4096u) : "memory", "m0");
        // the aligned dword that holds this lane's scale
        const uintptr_t sa = (reinterpret_cast<uintptr_t>(p.k_scale) + ((size_t)(half ? ry : rx) + j) * KSZ) & ~(uintptr_t)3;
        asm volatile("s_mov_b32 m0, %1\n\t"
                     "s_nop 0\n\t"
                     "global_load_lds_dword %0, off"
                     :: "v"(sa), "s"(dst + (uint32_t)SC_PAIR_BYTES) : "memory", "m0");
    };
    request_pair(0, 0);
    if (npair > 1) request_pair(1, 1);

    // A operands.  Row i of operand 0 is head 32*((i>>2)&1) + 4*(i>>3) + (i&3), operand 1 adds 16:
    // with the 32x32 accumulator layout (row = 8*(r/4) + 4*half + r%4) lane (key, half) then holds
    // heads 32*half + r in register r of accumulator 0 and heads 32*half + 16 + r in accumulator 1.
    // The contraction runs over 16-byte chunks in the order 4*half + ks (ks = 0..3).
    i32x4 qa[NT][2][4];
#pragma unroll
    for (int s = 0; s < NT; ++s) {
        const int head0 = 32 * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);
        const int ts = t + (s < nt ? s : 0);                   // a unit of one token loads that token twice
        const int8_t *q0 = p.q + ((size_t)ts * LI_HEADS + head0) * LI_DIM + 64 * half;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            qa[s][0][ks] = *reinterpret_cast<const i32x4 *>(q0 + 16 * ks);
            qa[s][1][ks] = *reinterpret_cast<const i32x4 *>(q0 + 16 * LI_DIM + 16 * ks);
        }
    }
    // per-head factors: lane l computes head l's.  One token per wave: read back lane by lane they are
    // wave-uniform and sit in scalar registers.  Two tokens: they go to this wave's rows of wsc_lds and are
    // read as broadcasts, four heads at a time, along the head sum.
    // VAR = 1 keeps the fp16 query scales and weights of head pairs (2i, 2i+1) packed instead.
    static_assert(!(VAR && NT > 1), "the fp16 variant scores one token per wave");
    float wsc[(VAR || NT > 1) ? 1 : LI_HEADS];
    uint32_t qs2[VAR ? LI_HEADS / 2 : 1], w2[VAR ? LI_HEADS / 2 : 1];
    if (VAR) {
        const uint32_t mq = reinterpret_cast<const uint32_t *>(p.q_scale)[(size_t)t * (LI_HEADS / 2) + (l & 31)];
        const uint32_t mw = reinterpret_cast<const uint32_t *>(p.weight)[(size_t)t * (LI_HEADS / 2) + (l & 31)];
#pragma unroll
        for (int h = 0; h < LI_HEADS / 2; ++h) {
            qs2[h] = (uint32_t)__builtin_amdgcn_readlane((int)mq, h);
            w2[h] = (uint32_t)__builtin_amdgcn_readlane((int)mw, h);
        }
    } else if (NT > 1) {
#pragma unroll
        for (int s = 0; s < NT; ++s) wsc_lds[w][s][l] = w_scale_of(p, (size_t)(t + (s < nt ? s : 0)) * LI_HEADS + l);
    } else {
        const float mine = w_scale_of(p, (size_t)t * LI_HEADS + l);
#pragma unroll
        for (int h = 0; h < LI_HEADS; ++h) wsc[h] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), h));
    }

    float *srow0 = p.scores + (size_t)t * p.score_stride;
    float *smp0 = p.sample + (size_t)t * (p.score_stride / LI_SAMPLE_GROUP);
    // 2^-11 as a run-time value, so that it sits in a scalar register (the mix instructions take no literal)
    const float scale = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(0x3a000000));
    // this lane's operand chunks of row j inside a staged block
    int koff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) koff[ks] = j * LI_DIM + (((4 * half + ks) ^ (j & 7)) << 4);

    // One trip.  Requests complete in the order they were made, so "at most nine outstanding" (the
    // nine of the following pair; the score store of the previous trip may or may not be among them)
    // means that this trip's pair has landed.  Its operands and scale move to registers, which frees
    // the buffer for the pair two ahead; then the pair is scored.
    auto trip = [&](const int pr, const int buf) {
        const int8_t *src = &kstage[w][buf][0];
        i32x4 kx[4], ky[4];
        if (pr + 1 < npair) __builtin_amdgcn_s_waitcnt(0x0F79);  // vmcnt(9)
        else __builtin_amdgcn_s_waitcnt(0x0F70);                 // vmcnt(0)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            kx[ks] = *reinterpret_cast<const i32x4 *>(src + koff[ks]);
            ky[ks] = *reinterpret_cast<const i32x4 *>(src + 4096 + koff[ks]);
        }
        const uint32_t ksraw = *reinterpret_cast<const uint32_t *>(src + SC_PAIR_BYTES + 4 * l);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);                      // lgkmcnt(0): the buffer has been read
        if (pr + 2 < npair) request_pair(pr + 2, buf);
        float ksc;
        uint32_t ks2 = 0;                                        // the key's fp16 scale twice (VAR = 1)
        if (KDT == PTO_DT_FP32) {
            ksc = __uint_as_float(ksraw);
        } else {
            // rows of a block are 32 consecutive scales, so the parity of the lane's element follows j
            const int rrow = __builtin_amdgcn_readlane(run_row, 2 * pr + 0);
            const int rrow1 = __builtin_amdgcn_readlane(run_row, 2 * pr + 1);
            const bool odd = ((reinterpret_cast<uintptr_t>(p.k_scale) + ((size_t)(half ? rrow1 : rrow) + j) * KSZ) & 2) != 0;
            const uint16_t hbits = (uint16_t)(odd ? ksraw >> 16 : ksraw);
            ksc = KDT == PTO_DT_BF16 ? bf16_bits_to_f32(hbits) : (float)__builtin_bit_cast(_Float16, hbits);
            ks2 = (uint32_t)hbits | ((uint32_t)hbits << 16);
        }
        // the staged pair serves every token of the unit
        auto score_token = [&](auto s_tag, float *srow, float *smp) {
            constexpr int s = decltype(s_tag)::value;
            i32x16 ax0, ax1, ay0, ay1;
#pragma unroll
            for (int r = 0; r < 16; ++r) { ax0[r] = 0; ax1[r] = 0; ay0[r] = 0; ay1[r] = 0; }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                ax0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[s][0][ks], kx[ks], ax0, 0, 0, 0);
                ax1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[s][1][ks], kx[ks], ax1, 0, 0, 0);
                ay0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[s][0][ks], ky[ks], ay0, 0, 0, 0);
                ay1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[s][1][ks], ky[ks], ay1, 0, 0, 0);
            }
            // lo[o][i] / hi[o][i]: heads 16*o + 2*i, +1 (lo) and 32 + 16*o + 2*i, +1 (hi) of this lane's key
            uint32_t lo[2][8], hi[2][8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t x0 = VAR ? fp16_pair(ax0[2 * i], ax0[2 * i + 1], scale) : relu_fp16_pair(ax0[2 * i], ax0[2 * i + 1], scale);
                const uint32_t y0 = VAR ? fp16_pair(ay0[2 * i], ay0[2 * i + 1], scale) : relu_fp16_pair(ay0[2 * i], ay0[2 * i + 1], scale);
                const uint32_t x1 = VAR ? fp16_pair(ax1[2 * i], ax1[2 * i + 1], scale) : relu_fp16_pair(ax1[2 * i], ax1[2 * i + 1], scale);
                const uint32_t y1 = VAR ? fp16_pair(ay1[2 * i], ay1[2 * i + 1], scale) : relu_fp16_pair(ay1[2 * i], ay1[2 * i + 1], scale);
                const auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
                lo[0][i] = s0[0]; hi[0][i] = s0[1];
                lo[1][i] = s1[0]; hi[1][i] = s1[1];
            }
            float sum = 0.f;
            if (VAR) {
                const float one = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(0x3f800000));
#pragma unroll
                for (int o = 0; o < 2; ++o) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const uint32_t v = dequant_relu_weight(lo[o][i], qs2[8 * o + i], ks2, w2[8 * o + i]);
                        sum = __fadd_rn(sum, mul_f16_f32<0>(v, one));
                        sum = __fadd_rn(sum, mul_f16_f32<1>(v, one));
                    }
                }
#pragma unroll
                for (int o = 0; o < 2; ++o) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const uint32_t v = dequant_relu_weight(hi[o][i], qs2[16 + 8 * o + i], ks2, w2[16 + 8 * o + i]);
                        sum = __fadd_rn(sum, mul_f16_f32<0>(v, one));
                        sum = __fadd_rn(sum, mul_f16_f32<1>(v, one));
                    }
                }
                const int pos = key0 + 64 * pr + l;
                if (pos < cur) srow[pos] = sum;
                if (sample_lane(pos, cur)) smp[pos >> 4] = sum;
                return;
            }
            if (NT > 1) {
                // heads ascending: lo[0][0..7], lo[1][0..7], hi[0][0..7], hi[1][0..7], two heads per register
                const f32x4 *wrow = reinterpret_cast<const f32x4 *>(&wsc_lds[w][s][0]);
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const f32x4 w4 = wrow[q];                        // heads 4q .. 4q+3, the same address on every lane
                    const int o = (q >> 2) & 1, i = 2 * (q & 3);
                    const uint32_t x0 = q < 8 ? lo[o][i] : hi[o][i], x1 = q < 8 ? lo[o][i + 1] : hi[o][i + 1];
                    sum = __fadd_rn(sum, mul_f16_f32_v<0>(x0, w4[0]));
                    sum = __fadd_rn(sum, mul_f16_f32_v<1>(x0, w4[1]));
                    sum = __fadd_rn(sum, mul_f16_f32_v<0>(x1, w4[2]));
                    sum = __fadd_rn(sum, mul_f16_f32_v<1>(x1, w4[3]));
                }
            } else {
#pragma unroll
                for (int o = 0; o < 2; ++o) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        sum = __fadd_rn(sum, mul_f16_f32<0>(lo[o][i], wsc[16 * o + 2 * i]));
                        sum = __fadd_rn(sum, mul_f16_f32<1>(lo[o][i], wsc[16 * o + 2 * i + 1]));
                    }
                }
#pragma unroll
                for (int o = 0; o < 2; ++o) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        sum = __fadd_rn(sum, mul_f16_f32<0>(hi[o][i], wsc[32 + 16 * o + 2 * i]));
                        sum = __fadd_rn(sum, mul_f16_f32<1>(hi[o][i], wsc[32 + 16 * o + 2 * i + 1]));
                    }
                }
            }
            const int pos = key0 + 64 * pr + l;
            const float sc = __fmul_rn(sum, ksc);
            if (pos < cur) srow[pos] = sc;
            if (sample_lane(pos, cur)) smp[pos >> 4] = sc;
        };
        score_token(std::integral_constant<int, 0>{}, srow0, smp0);
        if (NT > 1 && nt > 1)
            score_token(std::integral_constant<int, NT - 1>{}, srow0 + p.score_stride, smp0 + p.score_stride / LI_SAMPLE_GROUP);
    };
    for (int pr = 0; pr < npair; pr += 2) {
        trip(pr, 0);
        if (pr + 1 < npair) trip(pr + 1, 1);
    }
}

// ---------------------------------------------------------------------------------- select

constexpr int SEL_THREADS = 1024;
constexpr int SEL_WAVES = SEL_THREADS / 64;

// General select of one query token: every pass re-reads the score row (L2-resident) from memory.
// Slow (five passes over the row) but free of capacity assumptions; the fast kernel falls back to it.
// hist: >= 256 words, sortbuf: LI_MAX_SELECT entries, both in LDS.
__device__ void select_streaming(const LiParams &p, const int t, uint32_t *hist, unsigned long long *sortbuf)
{
    __shared__ uint32_t wave_gt[SEL_WAVES], wave_eq[SEL_WAVES];
    __shared__ uint32_t sh_prefix, sh_krem;

    const int b = t / p.S1;
    const int s = t - b * p.S1;
    const int tid = threadIdx.x;
    const int wv = tid >> 6;
    const int lane = tid & 63;
    int cur = p.act[b];
    const int cap = p.maxblk * p.bs;
    cur = cur < 0 ? 0 : (cur > cap ? cap : cur);
    int n = cur - (p.S1 - 1 - s);
    n = n < 0 ? 0 : n;
    const int k = p.k;
    const float *srow = p.scores + (size_t)t * p.score_stride;
    int32_t *out = p.topk_res + (size_t)t * k;

    // sort width: the next power of two that holds min(n, k) candidates
    const int nsel = n < k ? n : k;
    int width = 64;
    while (width < nsel) width <<= 1;
    for (int i = tid; i < width; i += SEL_THREADS) sortbuf[i] = 0ull;   // 0 sorts after every candidate

    if (n <= k) {
        __syncthreads();
        for (int i = tid; i < n; i += SEL_THREADS)
            sortbuf[i] = ((unsigned long long)score_key(srow[i]) << 32) | (uint32_t)(~(uint32_t)i);
    } else {
        // ---- radix select: after the passes, prefix = key of the k-th best and krem = how many
        // candidates with exactly that key are taken
        uint32_t prefix = 0, krem = (uint32_t)k;
        for (int pass = 0; pass < 4; ++pass) {
            const int shift = 24 - 8 * pass;
            for (int i = tid; i < 256; i += SEL_THREADS) hist[i] = 0;
            __syncthreads();
            const uint32_t himask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
            for (int i0 = 0; i0 < n; i0 += SEL_THREADS) {
                const int i = i0 + tid;
                bool active = false;
                uint32_t digit = 0;
                if (i < n) {
                    const uint32_t key = score_key(srow[i]);
                    active = (key & himask) == prefix;
                    digit = (key >> shift) & 0xffu;
                }
                // scores cluster: peel up to two digits shared by many lanes with one add each
                unsigned long long rem = __ballot(active);
#pragma unroll 1
                for (int peel = 0; peel < 2 && rem != 0ull; ++peel) {
                    const int first = __ffsll((long long)rem) - 1;
                    const uint32_t d = __shfl(digit, first);
                    const unsigned long long same = __ballot(active && digit == d) & rem;
                    if (__popcll(same) < 8) break;
                    if (lane == first) atomicAdd(&hist[d], (uint32_t)__popcll(same));
                    rem &= ~same;
                }
                if ((rem >> lane) & 1ull) atomicAdd(&hist[digit], 1u);
            }
            __syncthreads();
            if (tid < 64) {
                // bins in descending order: lane i owns bins 255-4i .. 252-4i
                uint32_t c[4];
                uint32_t tot = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) { c[e] = hist[255 - 4 * tid - e]; tot += c[e]; }
                uint32_t incl = tot;
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const uint32_t v = __shfl_up(incl, off);
                    if (lane >= off) incl += v;
                }
                uint32_t above = incl - tot;      // candidates in bins above this lane's four
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (above < krem && krem <= above + c[e]) {
                        sh_prefix = prefix | ((uint32_t)(255 - 4 * tid - e) << shift);
                        sh_krem = krem - above;
                    }
                    above += c[e];
                }
            }
            __syncthreads();
            prefix = sh_prefix;
            krem = sh_krem;
            __syncthreads();
        }
        const uint32_t thr = prefix;
        const uint32_t n_gt = (uint32_t)k - krem;

        // ---- compaction in position order: wave wv owns positions [wv*seg, (wv+1)*seg)
        const int seg = ((n + SEL_WAVES - 1) / SEL_WAVES + 63) / 64 * 64;
        const int lo = wv * seg;
        int hi = lo + seg;
        hi = hi > n ? n : hi;
        uint32_t cgt = 0, ceq = 0;
        for (int i0 = lo; i0 < hi; i0 += 64) {
            const int i = i0 + lane;
            uint32_t key = 0;
            if (i < hi) key = score_key(srow[i]);
            cgt += (uint32_t)__popcll(__ballot(i < hi && key > thr));
            ceq += (uint32_t)__popcll(__ballot(i < hi && key == thr));
        }
        if (lane == 0) { wave_gt[wv] = cgt; wave_eq[wv] = ceq; }
        __syncthreads();
        uint32_t base_gt = 0, base_eq = 0;
        for (int i = 0; i < wv; ++i) { base_gt += wave_gt[i]; base_eq += wave_eq[i]; }
        const unsigned long long lt_mask = (1ull << lane) - 1ull;
        for (int i0 = lo; i0 < hi; i0 += 64) {
            const int i = i0 + lane;
            uint32_t key = 0;
            if (i < hi) key = score_key(srow[i]);
            const bool gt = i < hi && key > thr;
            const bool eq = i < hi && key == thr;
            const unsigned long long mgt = __ballot(gt), meq = __ballot(eq);
            const unsigned long long comp = ((unsigned long long)key << 32) | (uint32_t)(~(uint32_t)i);
            if (gt) sortbuf[base_gt + (uint32_t)__popcll(mgt & lt_mask)] = comp;
            if (eq) {
                const uint32_t rank = base_eq + (uint32_t)__popcll(meq & lt_mask);
                if (rank < krem) sortbuf[n_gt + rank] = comp;
            }
            base_gt += (uint32_t)__popcll(mgt);
            base_eq += (uint32_t)__popcll(meq);
        }
    }
    __syncthreads();

    // ---- bitonic sort, descending on (key, ~position): score descending, position ascending
    for (int size = 2; size <= width; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = tid; i < (width >> 1); i += SEL_THREADS) {
                const int pos = 2 * i - (i & (stride - 1));
                const unsigned long long a = sortbuf[pos], c = sortbuf[pos + stride];
                const bool desc = (pos & size) == 0;
                if ((a < c) == desc) { sortbuf[pos] = c; sortbuf[pos + stride] = a; }
            }
            __syncthreads();
        }
    }
    for (int i = tid; i < k; i += SEL_THREADS)
        out[i] = i < nsel ? (int32_t)(~(uint32_t)(sortbuf[i] & 0xffffffffull)) : -1;
}


// ------------------------------------------------------------------ register-resident select

// descending bitonic sort of width (power of two, 64..2048) 64-bit keys in LDS, 1024 threads.
// Thread tid owns positions 2*tid and 2*tid+1: strides 1..64 are done in registers and wave shuffles,
// only strides >= 128 go through LDS with a barrier.
__device__ __forceinline__ unsigned long long shfl_xor_u64(const unsigned long long v, const int mask)
{
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask);
    const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask);
    return ((unsigned long long)hi << 32) | lo;
}

__device__ void bitonic_sort_desc(unsigned long long *buf, const int width, const int tid)
{
    const bool active = 2 * tid < width;
    unsigned long long e0 = 0ull, e1 = 0ull;
    if (active) { e0 = buf[2 * tid]; e1 = buf[2 * tid + 1]; }
    for (int size = 2; size <= width; size <<= 1) {
        const bool desc = ((2 * tid) & size) == 0;      // both positions of a thread share the direction bit (size >= 2)
        int stride = size >> 1;
        if (stride >= 128) {
            // cross-wave strides through LDS
            if (active) { buf[2 * tid] = e0; buf[2 * tid + 1] = e1; }
            __syncthreads();
            for (; stride >= 128; stride >>= 1) {
                for (int i = tid; i < (width >> 1); i += SEL_THREADS) {
                    const int pos = 2 * i - (i & (stride - 1));
                    const unsigned long long a = buf[pos], c = buf[pos + stride];
                    const bool d = (pos & size) == 0;
                    if ((a < c) == d) { buf[pos] = c; buf[pos + stride] = a; }
                }
                __syncthreads();
            }
            if (active) { e0 = buf[2 * tid]; e1 = buf[2 * tid + 1]; }
        }
        for (; stride >= 2; stride >>= 1) {
            // partner thread tid ^ (stride/2), same slot; the lower position keeps the max when descending
            const unsigned long long p0 = shfl_xor_u64(e0, stride >> 1);
            const unsigned long long p1 = shfl_xor_u64(e1, stride >> 1);
            const bool lower = ((2 * tid) & stride) == 0;
            const bool take_max = lower == desc;
            e0 = take_max ? (e0 > p0 ? e0 : p0) : (e0 < p0 ? e0 : p0);
            e1 = take_max ? (e1 > p1 ? e1 : p1) : (e1 < p1 ? e1 : p1);
        }
        {   // stride 1: the thread's own pair
            const unsigned long long hi = e0 > e1 ? e0 : e1, lo = e0 > e1 ? e1 : e0;
            e0 = desc ? hi : lo;
            e1 = desc ? lo : hi;
        }
    }
    if (active) { buf[2 * tid] = e0; buf[2 * tid + 1] = e1; }
    __syncthreads();
}

constexpr int SEL_SAMPLE = 4096;   // most keys sampled from a row
constexpr int SEL_CAP = 8192;      // candidates (keys above the pivot) the fast path holds in LDS
constexpr int SEL_STAGE = 4096;    // entries of the buckets down to the one holding the k-th best
constexpr int SEL_RANK_MAX = 512;  // rows of at most k keys: ordered by counting up to this length, else sorted

// how many entries of list[beg, end) are larger than e; eight LDS reads in flight per round
__device__ __forceinline__ uint32_t count_greater(const unsigned long long *list, const uint32_t beg, const uint32_t end,
                                                  const unsigned long long e)
{
    uint32_t rank = 0;
    for (uint32_t j0 = beg; j0 < end; j0 += 8) {
        unsigned long long x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = list[j0 + u < end ? j0 + u : end - 1];
#pragma unroll
        for (int u = 0; u < 8; ++u) rank += (j0 + u < end && x[u] > e) ? 1u : 0u;
    }
    return rank;
}

// the 64-bit word whose descending order is (score descending, position ascending); never zero
__device__ __forceinline__ unsigned long long order_word(const float score, const uint32_t pos)
{
    return ((unsigned long long)score_key(score) << 32) | (uint32_t)(~pos);
}

// score whose order-preserving image is key (the inverse of score_key)
__device__ __forceinline__ float key_score(const uint32_t key)
{
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

constexpr int SEL_SBINS = 1024;    // bins of the sample histogram
constexpr int SEL_BUCKETS = 2048;  // buckets the candidates are spread over
constexpr int SEL_WAVE_CAP = SEL_CAP / SEL_WAVES;   // candidates one wave can compact
constexpr int SEL_CHUNK = 32 * SEL_THREADS;   // scores one trip of the row scan holds in registers

// One workgroup per query token: a distribution-adaptive bucket select.  Every key is ordered by the
// word (score image << 32) | ~position, a strict order, so ties need no special case.
//   1. up to 4096 scores are sampled: the score kernel left one score of every 16 positions (which of
//      the 16, a hash of the group number decides) in a compact array.  A histogram of the
//      sample over [sample min, sample max] gives the pivot: the lower edge of the bin in which the
//      sample reaches rank r = r0 + 6*sqrt(r0) + 8, r0 = k*S/n.  With overwhelming probability at
//      least k and at most SEL_CAP scores of the row lie at or above it;
//   2. one pass over the row (32 scores per thread in flight at once, requested before the sample is
//      looked at) compacts the keys at or above the pivot into a candidate list;
//   3. the candidates are spread over 2048 buckets linear in the score between the pivot and the
//      sample maximum, bucket 0 highest: bins follow the values instead of the float encoding, so
//      the counters see few collisions and buckets stay short whatever the scale of the scores;
//   4. a prefix sum over the bucket counts finds the bucket holding the k-th best key; the buckets
//      down to it are staged contiguously and each is ordered by counting (a key's rank = the number
//      of larger keys of its bucket).  Output slots below k are written straight to memory.
// If the pivot misjudges the row (fewer than k candidates, more than the list holds, or a bucket
// range too long to stage) the general streaming select runs instead.
__global__ __launch_bounds__(SEL_THREADS) void li_select_kernel(const LiParams p)
{
    __shared__ unsigned long long cand[SEL_CAP + 64];  // + one dump slot per lane
    __shared__ unsigned long long stage[SEL_STAGE];    // also the sort buffer of the other paths
    __shared__ uint16_t sbucket[SEL_STAGE];            // bucket of every staged entry
    __shared__ uint32_t bcount[SEL_BUCKETS];
    __shared__ uint32_t boff[SEL_BUCKETS];
    __shared__ uint32_t shist[SEL_SBINS];
    __shared__ uint32_t hist[256];                     // streaming path only
    __shared__ uint32_t wave_tot[SEL_WAVES];
    __shared__ float wave_mn[SEL_WAVES], wave_mx[SEL_WAVES];
    __shared__ uint32_t sh_over, sh_tb;

    const int t = blockIdx.x;
    const int b = t / p.S1;
    const int s = t - b * p.S1;
    const int tid = threadIdx.x;
    const int wv = tid >> 6;
    const int lane = tid & 63;
    int cur = p.act[b];
    const int cap = p.maxblk * p.bs;
    cur = cur < 0 ? 0 : (cur > cap ? cap : cur);
    int n = cur - (p.S1 - 1 - s);
    n = n < 0 ? 0 : n;
    const int k = p.k;
    const float *srow = p.scores + (size_t)t * p.score_stride;
    int32_t *out = p.topk_res + (size_t)t * k;

    if (n <= k) {
        // everything is selected; the tail of the output row is padding
        for (int i = n + tid; i < k; i += SEL_THREADS) out[i] = -1;
        if (n > SEL_RANK_MAX) {
            int width = 64;
            while (width < n) width <<= 1;
            for (int i = tid; i < width; i += SEL_THREADS) stage[i] = i < n ? order_word(srow[i], (uint32_t)i) : 0ull;
            __syncthreads();
            bitonic_sort_desc(stage, width, tid);
            for (int i = tid; i < n; i += SEL_THREADS) out[i] = (int32_t)(~(uint32_t)stage[i]);
        } else {
            for (int i = tid; i < n; i += SEL_THREADS) stage[i] = order_word(srow[i], (uint32_t)i);
            __syncthreads();
            for (int i = tid; i < n; i += SEL_THREADS) {
                const unsigned long long e = stage[i];
                out[count_greater(stage, 0u, (uint32_t)n, e)] = (int32_t)(~(uint32_t)e);
            }
        }
        return;
    }

    // ---- 1. sample: the loads go out first, then the first chunk of the row, so that one memory
    // latency covers both
    // (the score kernel left one score of every 16 positions in a compact array; a row longer than
    // 16 * SEL_SAMPLE takes every other one).  Rows with hardly any full group go the general way.
    const uint32_t s_full = (uint32_t)n / (uint32_t)LI_SAMPLE_GROUP;
    if (s_full < 64u) {
        select_streaming(p, t, hist, stage);                     // uniform: the whole workgroup goes
        return;
    }
    const uint32_t sstep = s_full > (uint32_t)SEL_SAMPLE ? 2u : 1u;
    const uint32_t S = s_full / sstep;
    constexpr int SPT = SEL_SAMPLE / SEL_THREADS;
    const float *smp = p.sample + (size_t)t * (p.score_stride / LI_SAMPLE_GROUP);
    float sx[SPT];
    bool sval[SPT];
#pragma unroll
    for (int e = 0; e < SPT; ++e) {
        const uint32_t i = (uint32_t)(tid + e * SEL_THREADS);
        sval[e] = i < S;
        sx[e] = smp[(sval[e] ? i : 0u) * sstep];
    }
    // the row as 16-byte vectors: thread tid holds vectors u*1024 + tid of a chunk.  The row buffer is
    // score_stride (a multiple of 32) long, so whole vectors stay inside it.
    const int last_vec = (int)(p.score_stride >> 2) - 1;
    auto load_chunk = [&](const int c0, f32x4 (&v)[8]) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int vi = (c0 >> 2) + u * SEL_THREADS + tid;
            v[u] = reinterpret_cast<const f32x4 *>(srow)[vi < last_vec ? vi : last_vec];
        }
    };
    f32x4 v[8], vn[8];
    load_chunk(0, v);

    for (int i = tid; i < SEL_SBINS; i += SEL_THREADS) shist[i] = 0u;
    for (int i = tid; i < SEL_BUCKETS; i += SEL_THREADS) bcount[i] = 0u;
    if (tid == 0) sh_over = 0u;
    {
        float mn = __builtin_inff(), mx = -__builtin_inff();
#pragma unroll
        for (int e = 0; e < SPT; ++e)
            if (sval[e]) { mn = fminf(mn, sx[e]); mx = fmaxf(mx, sx[e]); }
        mn = wave_min(mn);
        mx = wave_max(mx);
        if (lane == 0) { wave_mn[wv] = mn; wave_mx[wv] = mx; }
    }
    __syncthreads();
    float smin = wave_mn[0], smax = wave_mx[0];
#pragma unroll
    for (int i = 1; i < SEL_WAVES; ++i) { smin = fminf(smin, wave_mn[i]); smax = fmaxf(smax, wave_mx[i]); }
    const uint32_t r0 = ((uint32_t)k * S + (uint32_t)n - 1u) / (uint32_t)n;
    const uint32_t r = r0 + (uint32_t)(6.0f * __builtin_sqrtf((float)r0)) + 8u;
    float pivot = -__builtin_inff();       // candidates: score >= pivot
    float blo = smin;                      // lower edge of the lowest bucket
    if (r < S) {
        const float range = smax - smin;
        const float sscale = range > 0.f ? (float)SEL_SBINS / range : 0.f;
#pragma unroll
        for (int e = 0; e < SPT; ++e) {
            if (sval[e]) {
                const uint32_t sb = (uint32_t)fmaxf((sx[e] - smin) * sscale, 0.f);
                atomicAdd(&shist[sb < (uint32_t)SEL_SBINS ? sb : (uint32_t)SEL_SBINS - 1u], 1u);
            }
        }
        __syncthreads();
        // every wave scans the 1024 bins from the top by itself (lane l owns the 16 bins below
        // 1024 - 16*l): the bin in which the running count reaches r
        uint32_t c[16];
        uint32_t tot = 0;
        {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(&shist[SEL_SBINS - 16 - 16 * lane]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u32x4 x = src[q];
                c[4 * q] = x[0]; c[4 * q + 1] = x[1]; c[4 * q + 2] = x[2]; c[4 * q + 3] = x[3];
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) tot += c[q];
        }
        uint32_t before = wave_incl_scan(tot) - tot;
        uint32_t pb = 0;                   // found by exactly one lane (the sample holds S >= r scores)
#pragma unroll
        for (int q = 15; q >= 0; --q) {
            if (before < r && r <= before + c[q]) pb = (uint32_t)(SEL_SBINS - 16 - 16 * lane + q);
            before += c[q];
        }
        pb = wave_max_u32(pb);
        pivot = smin + (float)pb * (range * (1.0f / (float)SEL_SBINS));
        blo = pivot;
    }
    // the buckets reach a quarter of the range past the sample maximum, so that the few scores above
    // it spread out too; anything beyond shares bucket 0
    const float bscale = smax - blo > 0.f ? (float)SEL_BUCKETS / (1.25f * (smax - blo)) : 0.f;

    // ---- 2. candidates.  Wave w compacts the candidates among its keys into its own region of the
    // list, cand[w*SEL_WAVE_CAP ...], so the waves share no counter.  A key costs a compare and an add
    // to be counted and, branch-free, a compare, a select, an add and one LDS write of the raw
    // (score bits, position) pair: a key that is no candidate goes to the lane's dump slot.  The
    // order word is formed later, for the candidates only.  Wave-wide sums use DPP, not LDS.
    uint32_t wave_count = 0;               // candidates of this wave so far (uniform)
    auto scan_chunk = [&](const int c0, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;          // the whole chunk lies inside the row
        const int i_base = c0 + 4 * tid;
        uint32_t mine = 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int i = i_base + 4 * u * SEL_THREADS + c;
                mine += ((FULL || i < n) && v[u][c] >= pivot) ? 1u : 0u;
            }
        }
        const uint32_t incl = wave_incl_scan(mine);
        const uint32_t wave_n = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        if (wave_count + wave_n > (uint32_t)SEL_WAVE_CAP) {       // region overflow: the streaming path will run
            if (lane == 0) sh_over = 1u;
            return;
        }
        uint32_t slot = (uint32_t)(wv * SEL_WAVE_CAP) + wave_count + incl - mine;
        wave_count += wave_n;
        const uint32_t dump = (uint32_t)(SEL_CAP + lane);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int i = i_base + 4 * u * SEL_THREADS + c;
                const bool is_c = (FULL || i < n) && v[u][c] >= pivot;
                cand[is_c ? slot : dump] = ((unsigned long long)(uint32_t)i << 32) | __float_as_uint(v[u][c]);
                slot += is_c ? 1u : 0u;
            }
        }
    };
    for (int c0 = 0; c0 < n; c0 += SEL_CHUNK) {
        if (c0 + SEL_CHUNK < n) load_chunk(c0 + SEL_CHUNK, vn);
        if (c0 + SEL_CHUNK <= n) scan_chunk(c0, std::true_type{});
        else scan_chunk(c0, std::false_type{});
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = vn[u];
    }
    if (lane == 0) wave_tot[wv] = wave_count;

    // ---- 3. bucket of every candidate of the wave's own region (up to eight per lane) and its slot
    // inside the bucket
    constexpr int CPT = SEL_WAVE_CAP / 64;
    unsigned long long ce[CPT];
    uint32_t cb[CPT], cslot[CPT];
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const uint32_t j = (uint32_t)(u * 64 + lane);
        const unsigned long long raw = cand[wv * SEL_WAVE_CAP + (j < wave_count ? j : 0u)];
        ce[u] = j < wave_count ? order_word(__uint_as_float((uint32_t)raw), (uint32_t)(raw >> 32)) : 0ull;
    }
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const uint32_t lin = (uint32_t)fmaxf((key_score((uint32_t)(ce[u] >> 32)) - blo) * bscale, 0.f);
        cb[u] = (uint32_t)SEL_BUCKETS - 1u - (lin < (uint32_t)SEL_BUCKETS ? lin : (uint32_t)SEL_BUCKETS - 1u);
        cslot[u] = 0u;
        if ((uint32_t)(u * 64 + lane) < wave_count) cslot[u] = atomicAdd(&bcount[cb[u]], 1u);
    }
    __syncthreads();
    uint32_t n_cand = 0;
#pragma unroll
    for (int i = 0; i < SEL_WAVES; ++i) n_cand += wave_tot[i];
    if (sh_over != 0u || n_cand < (uint32_t)k) {
        __syncthreads();                                         // wave_tot is reused below
        select_streaming(p, t, hist, stage);                     // uniform: the whole workgroup goes
        return;
    }

    // ---- 4. bucket offsets (two buckets per thread) and the bucket holding the k-th best key
    {
        const uint32_t b0 = 2u * (uint32_t)tid;
        const uint32_t c0 = bcount[b0], c1 = bcount[b0 + 1u];
        const uint32_t tot = c0 + c1;
        const uint32_t incl = wave_incl_scan(tot);
        __syncthreads();                                         // every wave has read the candidate counts
        if (lane == 63) wave_tot[wv] = incl;
        __syncthreads();
        uint32_t before = incl - tot;
#pragma unroll
        for (int i = 0; i < SEL_WAVES; ++i) before += i < wv ? wave_tot[i] : 0u;
        boff[b0] = before;
        boff[b0 + 1u] = before + c0;
        if (before < (uint32_t)k && (uint32_t)k <= before + c0) sh_tb = b0;
        else if (before + c0 < (uint32_t)k && (uint32_t)k <= before + tot) sh_tb = b0 + 1u;
    }
    __syncthreads();
    const uint32_t tb = sh_tb;
    const uint32_t n_stage = boff[tb] + bcount[tb];
    if (n_stage > (uint32_t)SEL_STAGE) {
        __syncthreads();
        select_streaming(p, t, hist, stage);
        return;
    }
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        if ((uint32_t)(u * 64 + lane) < wave_count && cb[u] <= tb) {
            const uint32_t idx = boff[cb[u]] + cslot[u];
            stage[idx] = ce[u];
            sbucket[idx] = (uint16_t)cb[u];
        }
    }
    __syncthreads();
    // Order inside buckets by counting.  Neighbouring threads take neighbouring staged entries, which
    // mostly share a bucket, so the loop lengths of a wave agree and its LDS reads are broadcasts; a
    // thread's two entries are ranked side by side, four keys of each bucket per trip, to keep eight
    // reads in flight.  Entries past the first 2048 (the tail of the last bucket) take a second trip
    // that only the waves holding them make.
    for (uint32_t i0 = 0; i0 < n_stage; i0 += 2 * SEL_THREADS) {
        if (i0 + (uint32_t)(wv * 64) >= n_stage) break;          // wave-uniform: nothing staged for this wave
        unsigned long long e[2];
        uint32_t beg[2], len[2], rank[2];
        uint32_t maxlen = 0;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t i = i0 + (uint32_t)(q * SEL_THREADS + tid);
            const bool ok = i < n_stage;
            e[q] = stage[ok ? i : 0u];
            const uint32_t bk = sbucket[ok ? i : 0u];
            beg[q] = boff[bk];
            len[q] = ok ? bcount[bk] : 0u;
            rank[q] = 0u;
            maxlen = len[q] > maxlen ? len[q] : maxlen;
        }
        for (uint32_t j = 0; j < maxlen; j += 4) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
#pragma unroll
                for (uint32_t d = 0; d < 4; ++d) {
                    const bool in = j + d < len[q];
                    const unsigned long long x = stage[in ? beg[q] + j + d : 0u];
                    rank[q] += (in && x > e[q]) ? 1u : 0u;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t fin = beg[q] + rank[q];
            if (i0 + (uint32_t)(q * SEL_THREADS + tid) < n_stage && fin < (uint32_t)k) out[fin] = (int32_t)(~(uint32_t)e[q]);
        }
    }
}

__global__ __launch_bounds__(SEL_THREADS) void li_select_stream_kernel(const LiParams p)
{
    __shared__ uint32_t hist[256];
    __shared__ unsigned long long sortbuf[LI_MAX_SELECT];
    select_streaming(p, (int)blockIdx.x, hist, sortbuf);
}

}  // namespace

hipError_t li_launch(const LiParams &p, hipStream_t stream)
{
    const dim3 block(256);
    const int nt = p.nt;
    const int nunits = p.B * ((p.S1 + nt - 1) / nt);
    dim3 grid;
    if (p.balanced) {
        grid = dim3((unsigned)p.score_wgs);
    } else {
        const unsigned gx = (unsigned)((p.score_stride + 4 * p.ppw * 64 - 1) / (4 * p.ppw * 64));
        grid = dim3(gx, (unsigned)nunits);
    }
    if (p.variant == 1) hipLaunchKernelGGL((li_score_kernel<PTO_DT_FP16, 1>), grid, block, 0, stream, p);
    else if (nt == 2) {
        if (p.k_dt == PTO_DT_FP32) hipLaunchKernelGGL((li_score_kernel<PTO_DT_FP32, 0, 2>), grid, block, 0, stream, p);
        else if (p.k_dt == PTO_DT_FP16) hipLaunchKernelGGL((li_score_kernel<PTO_DT_FP16, 0, 2>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((li_score_kernel<PTO_DT_BF16, 0, 2>), grid, block, 0, stream, p);
    } else {
        if (p.k_dt == PTO_DT_FP32) hipLaunchKernelGGL(li_score_kernel<PTO_DT_FP32>, grid, block, 0, stream, p);
        else if (p.k_dt == PTO_DT_FP16) hipLaunchKernelGGL(li_score_kernel<PTO_DT_FP16>, grid, block, 0, stream, p);
        else hipLaunchKernelGGL(li_score_kernel<PTO_DT_BF16>, grid, block, 0, stream, p);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(li_select_kernel, dim3((unsigned)p.T), dim3(SEL_THREADS), 0, stream, p);
    return hipGetLastError();
}

}  // namespace pto
