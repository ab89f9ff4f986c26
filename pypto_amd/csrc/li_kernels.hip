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
//                     one wave per run of 32-key blocks: v_mfma_i32_32x32x32_i8 with A = the
//                     token's 64 query heads (two 32-row operands resident in registers) and
//                     B = 32 key rows loaded straight from the paged cache in operand layout;
//                     epilogue in registers; scores to a [T, max_seq] fp32 workspace
//   li_select_kernel  one workgroup per query token, keys ordered by the strict word
//                     (score image << 32 | ~position): a histogram of a 2048-score sample gives a
//                     pivot, one pass over the row compacts the keys above it, those are spread over
//                     2048 buckets linear in the score and ordered inside buckets by counting;
//                     select_streaming (radix select over the row in memory + bitonic sort) is the
//                     capacity-free form it falls back to
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

// relu, scale by 2^-11, round to fp16, back to fp32
__device__ __forceinline__ float relu_fp16_term(const int dot)
{
    const float r = (float)(dot > 0 ? dot : 0) * (1.0f / 2048.0f);
    return (float)(_Float16)r;
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

__global__ __launch_bounds__(256) void li_score_kernel(const LiParams p)
{
    __shared__ float wsh[4][LI_HEADS];
    const int t = blockIdx.y;
    const int b = t / p.S1;
    int cur = p.act[b];
    const int cap = p.maxblk * p.bs;
    cur = cur < 0 ? 0 : (cur > cap ? cap : cur);
    const int w = threadIdx.x >> 6;
    const int l = threadIdx.x & 63;
    const int j = l & 31;
    const int half = l >> 5;
    const int key0 = (blockIdx.x * 4 + w) * (p.bpw * 32);
    if (key0 >= cur) return;
    int nblk = (cur - key0 + 31) >> 5;
    nblk = nblk > p.bpw ? p.bpw : nblk;

    // A operands.  Row i of operand 0 is head 32*((i>>2)&1) + 4*(i>>3) + (i&3), operand 1 adds 16:
    // with the 32x32 accumulator layout (row = 8*(r/4) + 4*half + r%4) lane (key, half) then holds
    // heads 32*half + r in register r of accumulator 0 and heads 32*half + 16 + r in accumulator 1.
    // The contraction is taken in the order bytes [64*half + 16*ks, +16) so that a lane's four key
    // loads are one contiguous 64-byte run.
    i32x4 qa[2][4];
    {
        const int head0 = 32 * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);
        const int8_t *q0 = p.q + ((size_t)t * LI_HEADS + head0) * LI_DIM + 64 * half;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            qa[0][ks] = *reinterpret_cast<const i32x4 *>(q0 + 16 * ks);
            qa[1][ks] = *reinterpret_cast<const i32x4 *>(q0 + 16 * LI_DIM + 16 * ks);
        }
    }
    // per-head factors: lane l computes head l's, the wave shares them through its LDS slice
    float wsc[32];
    {
        wsh[w][l] = w_scale_of(p, (size_t)t * LI_HEADS + l);
        const f32x4 *src = reinterpret_cast<const f32x4 *>(&wsh[w][32 * half]);
#pragma unroll
        for (int r4 = 0; r4 < 8; ++r4) {
            const f32x4 v = src[r4];
            wsc[4 * r4] = v[0]; wsc[4 * r4 + 1] = v[1]; wsc[4 * r4 + 2] = v[2]; wsc[4 * r4 + 3] = v[3];
        }
    }

    // key rows of block blk of this wave: 32 consecutive positions never straddle a page
    auto block_row = [&](const int blk) -> size_t {
        const int pos0 = key0 + 32 * blk;
        const int page = pos0 / p.bs;
        int pb = p.bt[(size_t)b * p.maxblk + page];
        pb = pb < 0 ? 0 : (pb >= p.nblocks ? p.nblocks - 1 : pb);
        return (size_t)pb * p.bs + (pos0 - page * p.bs) + j;
    };
    i32x4 kf[4], kn[4];
    float ksc, kscn;
    {
        const size_t row = block_row(0);
        const int8_t *kp = p.kcache + row * LI_DIM + 64 * half;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) kf[ks] = *reinterpret_cast<const i32x4 *>(kp + 16 * ks);
        ksc = load_scalar(p.k_scale, row, p.k_dt);
    }

    float *srow = p.scores + (size_t)t * p.score_stride;
    for (int blk = 0; blk < nblk; ++blk) {
        {   // next block's rows are in flight while this one is scored (the last iteration reloads itself)
            const size_t row = block_row(blk + 1 < nblk ? blk + 1 : blk);
            const int8_t *kp = p.kcache + row * LI_DIM + 64 * half;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) kn[ks] = *reinterpret_cast<const i32x4 *>(kp + 16 * ks);
            kscn = load_scalar(p.k_scale, row, p.k_dt);
        }
        i32x16 acc0, acc1;
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc0[r] = 0; acc1[r] = 0; }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[0][ks], kf[ks], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(qa[1][ks], kf[ks], acc1, 0, 0, 0);
        }
        float prod[32];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            prod[r] = __fmul_rn(wsc[r], relu_fp16_term(acc0[r]));
            prod[16 + r] = __fmul_rn(wsc[16 + r], relu_fp16_term(acc1[r]));
        }
        // heads 0..31 are summed by the lower half-wave, whose partial sum then seeds heads 32..63
        // in the upper half-wave: the chain is the sequential sum h = 0..63.
        float lo = 0.f;
#pragma unroll
        for (int r = 0; r < 32; ++r) lo = __fadd_rn(lo, prod[r]);
        float hi = __shfl(lo, j);
#pragma unroll
        for (int r = 0; r < 32; ++r) hi = __fadd_rn(hi, prod[r]);
        const int pos = key0 + 32 * blk + j;
        if (half == 1 && pos < cur) srow[pos] = __fmul_rn(hi, ksc);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) kf[ks] = kn[ks];
        ksc = kscn;
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

constexpr int SEL_SAMPLE = 2048;   // most keys sampled from a row
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
//   1. up to 2048 scores are sampled (one per stratum of the row, jittered).  A histogram of the
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
    const uint32_t S = n < SEL_SAMPLE ? (uint32_t)n : (uint32_t)SEL_SAMPLE;
    float sx[2];
    bool sval[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const uint32_t i = (uint32_t)(tid + e * SEL_THREADS);
        sval[e] = i < S;
        // stratum i of the row is [i*n/S, (i+1)*n/S): products stay below 2^28
        const uint32_t ic = sval[e] ? i : 0u;
        const uint32_t lo = ic * (uint32_t)n / S, hi = (ic + 1u) * (uint32_t)n / S;
        sx[e] = srow[lo + ((ic * 2654435761u) >> 16) % (hi - lo)];
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
        for (int e = 0; e < 2; ++e)
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
        for (int e = 0; e < 2; ++e) {
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
    const unsigned gx = (unsigned)((p.score_stride + 4 * p.bpw * 32 - 1) / (4 * p.bpw * 32));
    hipLaunchKernelGGL(li_score_kernel, dim3(gx, (unsigned)p.T), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(li_select_kernel, dim3((unsigned)p.T), dim3(SEL_THREADS), 0, stream, p);
    return hipGetLastError();
}

}  // namespace pto
