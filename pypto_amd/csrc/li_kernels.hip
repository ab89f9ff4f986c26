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
//   li_select_kernel  one workgroup per query token, score keys resident in registers: 3-pass radix
//                     select (11+11+10 bits) on an order-preserving 32-bit image of the score, a
//                     position select among candidates tied at the threshold, bitonic sort of the
//                     survivors by (score desc, position asc); li_select_stream_kernel is the
//                     memory-streaming form for rows longer than 65536
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

constexpr int HIST_BITS = 13;                 // first-level histogram: the top 13 bits of the key
constexpr int HIST_BINS = 1 << HIST_BITS;

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

constexpr int SEL_CAP = 4096;       // keys of the threshold bin the fast path holds in LDS
constexpr int SEL_RANK_MAX = 512;   // longest bin segment ordered by counting; longer ones use the bitonic sort
constexpr int SEL_DIRECT_MAX = 256; // most threshold-bin keys resolved by counting instead of radix passes

// One workgroup per query token.
//   pass 1 over the row: histogram of the top 13 key bits (LDS) -> the bin holding the k-th best key,
//           how many keys to take inside it, and the output offset of every bin above it;
//   pass 2 over the row: keys above that bin are scattered straight into their bin's output range,
//           keys inside it go to a candidate list;
//   candidates: few -> ordered by counting; many -> two 10-bit radix passes for the exact key of the
//           k-th best plus, if more candidates tie at that key than are needed, two passes over
//           their positions (lowest positions win);
//   each bin's range is then ordered by counting (every key counts the larger keys of its range).
// Order is (key desc, position asc) throughout: the 64-bit word (key << 32) | ~position, descending.
// A threshold bin with more than SEL_CAP keys takes the general streaming path.
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

__global__ __launch_bounds__(SEL_THREADS) void li_select_kernel(const LiParams p)
{
    __shared__ uint32_t hist[HIST_BINS];      // keys per first-level bin
    __shared__ uint32_t rhist[1024];          // histogram of the radix passes over the candidates
    __shared__ uint32_t cursor[HIST_BINS];    // next free output slot of each bin above the threshold bin
    __shared__ unsigned long long stage[LI_MAX_SELECT];   // survivors grouped by bin, unordered inside
    __shared__ unsigned long long sortbuf[LI_MAX_SELECT];
    __shared__ unsigned long long cand[SEL_CAP];
    __shared__ uint32_t wave_tot[SEL_WAVES];
    __shared__ uint32_t sh_prefix, sh_krem, sh_ncand, sh_nsurv, sh_longest;

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
    const int nsel = n < k ? n : k;

    // histogram of `digit` over the lanes with `act`; a digit shared by all of them costs one add
    auto hist_add = [&](uint32_t *h, const bool act, const uint32_t digit) {
        const unsigned long long m = __ballot(act);
        if (m == 0ull) return;
        const int first = __ffsll((long long)m) - 1;
        const uint32_t d = __shfl(digit, first);
        if (__ballot(act && digit == d) == m) {
            if (lane == first) atomicAdd(&h[d], (uint32_t)__popcll(m));
        } else if (act) {
            atomicAdd(&h[digit], 1u);
        }
    };
    // Bins of hist[] visited from the top (descending) or the bottom, eight per thread; finds the bin
    // holding the krem-th element and how many remain to be taken inside it.  nbins <= 8192.
    // With offsets != nullptr also records, for every bin, how many elements precede it.
    auto pick_bin = [&](const uint32_t *h, const int nbins, const bool descending, const uint32_t krem, uint32_t &bin,
                        uint32_t &rest, uint32_t *offsets) {
        uint32_t c[8];
        int idx[8];
        uint32_t tot = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int v = 8 * tid + e;                        // visiting order
            idx[e] = descending ? nbins - 1 - v : v;
            c[e] = v < nbins ? h[idx[e]] : 0u;
            tot += c[e];
        }
        uint32_t incl = tot;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t v = __shfl_up(incl, off);
            if (lane >= off) incl += v;
        }
        if (lane == 63) wave_tot[wv] = incl;
        __syncthreads();
        uint32_t before = incl - tot;
        for (int i = 0; i < wv; ++i) before += wave_tot[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (offsets != nullptr && 8 * tid + e < nbins) offsets[idx[e]] = before;
            if (before < krem && krem <= before + c[e]) { sh_prefix = (uint32_t)idx[e]; sh_krem = krem - before; }
            before += c[e];
        }
        __syncthreads();
        bin = sh_prefix;
        rest = sh_krem;
        __syncthreads();
    };

    if (tid == 0) { sh_ncand = 0; sh_nsurv = 0; sh_longest = 0; }
    if (n <= k) {
        // everything is selected: one range, ordered below
        for (int i = tid; i < n; i += SEL_THREADS)
            stage[i] = ((unsigned long long)score_key(srow[i]) << 32) | (uint32_t)(~(uint32_t)i);
        __syncthreads();
        if (n > SEL_RANK_MAX) {
            int width = 64;
            while (width < n) width <<= 1;
            for (int i = tid; i < width; i += SEL_THREADS) sortbuf[i] = i < n ? stage[i] : 0ull;
            __syncthreads();
            bitonic_sort_desc(sortbuf, width, tid);
        } else {
            for (int i = tid; i < n; i += SEL_THREADS) {
                const unsigned long long e = stage[i];
                sortbuf[count_greater(stage, 0u, (uint32_t)n, e)] = e;
            }
            __syncthreads();
        }
    } else {
        // Both passes over the row are rolled loops (the kernel runs once per token, so straight-line
        // code would be fetched cold) with the next round's eight loads in flight while a round is
        // processed.
        constexpr int U = 8;
        auto load_round = [&](const int i0, float (&v)[U]) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = i0 + u * SEL_THREADS + tid;
                v[u] = srow[i < n ? i : n - 1];
            }
        };
        // ---- pass 1: first-level histogram
        for (int i = tid; i < HIST_BINS; i += SEL_THREADS) hist[i] = 0u;
        __syncthreads();
        {
            float v[U], vn[U];
            load_round(0, v);
            for (int i0 = 0; i0 < n; i0 += SEL_THREADS * U) {
                load_round(i0 + SEL_THREADS * U, vn);
#pragma unroll
                for (int u = 0; u < U; ++u)
                    hist_add(hist, i0 + u * SEL_THREADS + tid < n, score_key(v[u]) >> (32 - HIST_BITS));
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = vn[u];
            }
        }
        __syncthreads();
        uint32_t bin0, rest;
        pick_bin(hist, HIST_BINS, true, (uint32_t)k, bin0, rest, cursor);
        const uint32_t n_bin = hist[bin0];
        const uint32_t base0 = (uint32_t)k - rest;               // first output slot of the threshold bin
        // longest range above the threshold bin (decides how the ranges are ordered)
        {
            uint32_t mx = 0;
            for (int i = tid; i < HIST_BINS; i += SEL_THREADS)
                if ((uint32_t)i > bin0) mx = hist[i] > mx ? hist[i] : mx;
            if (mx > 0) atomicMax(&sh_longest, mx);
        }
        __syncthreads();
        if (n_bin > (uint32_t)SEL_CAP) {
            select_streaming(p, t, hist, sortbuf);               // uniform: the whole workgroup goes
            return;
        }
        // ---- pass 2: scatter
        {
            float v[U], vn[U];
            load_round(0, v);
            for (int i0 = 0; i0 < n; i0 += SEL_THREADS * U) {
                load_round(i0 + SEL_THREADS * U, vn);
                uint32_t ncand_lane = 0;
                unsigned long long cval[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int i = i0 + u * SEL_THREADS + tid;
                    const uint32_t key = score_key(v[u]);
                    const uint32_t kb = key >> (32 - HIST_BITS);
                    const unsigned long long val = ((unsigned long long)key << 32) | (uint32_t)(~(uint32_t)i);
                    if (i < n && kb > bin0) stage[atomicAdd(&cursor[kb], 1u)] = val;
                    const bool is_c = i < n && kb == bin0;
                    cval[u] = is_c ? val : 0ull;
                    ncand_lane += is_c ? 1u : 0u;
                }
                // threshold-bin keys of the whole wave take one counter update
                if (__ballot(ncand_lane != 0u) != 0ull) {
                    uint32_t incl = ncand_lane;
#pragma unroll
                    for (int off = 1; off < 64; off <<= 1) {
                        const uint32_t x = __shfl_up(incl, off);
                        if (lane >= off) incl += x;
                    }
                    const uint32_t wave_n = __shfl(incl, 63);
                    uint32_t basec = 0;
                    if (lane == 0) basec = atomicAdd(&sh_ncand, wave_n);
                    basec = __shfl(basec, 0) + incl - ncand_lane;
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (cval[u] != 0ull) { if (basec < (uint32_t)SEL_CAP) cand[basec] = cval[u]; ++basec; }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = vn[u];
            }
        }
        __syncthreads();
        const uint32_t n_cand = sh_ncand < (uint32_t)SEL_CAP ? sh_ncand : (uint32_t)SEL_CAP;   // == n_bin

        if (n_cand <= (uint32_t)SEL_DIRECT_MAX) {
            // few candidates: a candidate's rank among them is its place in the bin's output range
            for (uint32_t i = tid; i < n_cand; i += SEL_THREADS) {
                const unsigned long long e = cand[i];
                const uint32_t rank = count_greater(cand, 0u, n_cand, e);
                if (rank < rest) sortbuf[base0 + rank] = e;
            }
        } else {
            // ---- exact key of the k-th best among the candidates: the 32 - HIST_BITS low key bits in two
            // radix passes (10 bits, then the rest)
            uint32_t prefix = bin0 << (32 - HIST_BITS);
            uint32_t krem = rest;
            constexpr int LOW = 32 - HIST_BITS;
#pragma unroll 1
            for (int pass = 0; pass < 2; ++pass) {
                const int shift = pass == 0 ? LOW - 10 : 0;
                const int nbits = pass == 0 ? 10 : LOW - 10;
                for (int i = tid; i < 1024; i += SEL_THREADS) rhist[i] = 0;
                __syncthreads();
                const uint32_t himask = 0xffffffffu << (shift + nbits);
                for (uint32_t i0 = 0; i0 < n_cand; i0 += SEL_THREADS) {
                    const uint32_t i = i0 + tid;
                    const uint32_t key = i < n_cand ? (uint32_t)(cand[i] >> 32) : 0u;
                    hist_add(rhist, i < n_cand && (key & himask) == prefix, (key >> shift) & ((1u << nbits) - 1u));
                }
                __syncthreads();
                uint32_t bin;
                pick_bin(rhist, 1 << nbits, true, krem, bin, krem, nullptr);
                prefix |= bin << shift;
            }
            const uint32_t thr = prefix;
            // ---- ties at thr: the krem lowest positions (17 position bits: 9 high, 8 low)
            for (int i = tid; i < 512; i += SEL_THREADS) rhist[i] = 0;
            __syncthreads();
            for (uint32_t i0 = 0; i0 < n_cand; i0 += SEL_THREADS) {
                const uint32_t i = i0 + tid;
                const unsigned long long c = i < n_cand ? cand[i] : 0ull;
                hist_add(rhist, i < n_cand && (uint32_t)(c >> 32) == thr, (~(uint32_t)c) >> 8);
            }
            __syncthreads();
            uint32_t hi_bin, lo_bin, rest2;
            pick_bin(rhist, 512, false, krem, hi_bin, rest2, nullptr);
            for (int i = tid; i < 256; i += SEL_THREADS) rhist[i] = 0;
            __syncthreads();
            for (uint32_t i0 = 0; i0 < n_cand; i0 += SEL_THREADS) {
                const uint32_t i = i0 + tid;
                const unsigned long long c = i < n_cand ? cand[i] : 0ull;
                const uint32_t pos = ~(uint32_t)c;
                hist_add(rhist, i < n_cand && (uint32_t)(c >> 32) == thr && (pos >> 8) == hi_bin, pos & 255u);
            }
            __syncthreads();
            pick_bin(rhist, 256, false, rest2, lo_bin, rest2, nullptr);
            const uint32_t idx_max = (hi_bin << 8) | lo_bin;         // largest position taken among the ties
            // ---- surviving candidates fill the threshold bin's range of the staging buffer
            for (uint32_t i0 = 0; i0 < n_cand; i0 += SEL_THREADS) {
                const uint32_t i = i0 + tid;
                const unsigned long long c = i < n_cand ? cand[i] : 0ull;
                const uint32_t key = (uint32_t)(c >> 32), pos = ~(uint32_t)c;
                const bool take = i < n_cand && (key > thr || (key == thr && pos <= idx_max));
                const unsigned long long m = __ballot(take);
                if (m != 0ull) {
                    uint32_t bs = 0;
                    const int first = __ffsll((long long)m) - 1;
                    if (lane == first) bs = atomicAdd(&sh_nsurv, (uint32_t)__popcll(m));
                    bs = __shfl(bs, first) + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
                    if (take && base0 + bs < (uint32_t)LI_MAX_SELECT) stage[base0 + bs] = c;
                }
            }
            if (tid == 0) atomicMax(&sh_longest, rest);              // this range is ordered like the others
        }
        __syncthreads();
        const bool direct = n_cand <= (uint32_t)SEL_DIRECT_MAX;      // threshold range already in sortbuf
        const uint32_t n_stage = direct ? base0 : (uint32_t)k;       // entries of stage[] to order
        if (sh_longest > (uint32_t)SEL_RANK_MAX) {
            // a long range: sort everything at once
            int width = 64;
            while (width < k) width <<= 1;
            for (int i = tid; i < width; i += SEL_THREADS) {
                unsigned long long e = 0ull;
                if ((uint32_t)i < n_stage) e = stage[i];
                else if (i < k) e = sortbuf[i];
                cand[i] = e;
            }
            __syncthreads();
            bitonic_sort_desc(cand, width, tid);
            for (int i = tid; i < k; i += SEL_THREADS) sortbuf[i] = cand[i];
            __syncthreads();
        } else {
            // ---- order every bin's range by counting
            for (uint32_t i = tid; i < n_stage; i += SEL_THREADS) {
                const unsigned long long e = stage[i];
                const uint32_t kb = (uint32_t)(e >> (64 - HIST_BITS));
                const uint32_t cnt = kb == bin0 ? rest : hist[kb];
                const uint32_t end = kb == bin0 ? (uint32_t)k : cursor[kb];
                const uint32_t beg = end - cnt;
                sortbuf[beg + count_greater(stage, beg, end, e)] = e;
            }
            __syncthreads();
        }
    }
    for (int i = tid; i < k; i += SEL_THREADS)
        out[i] = i < nsel ? (int32_t)(~(uint32_t)(sortbuf[i] & 0xffffffffull)) : -1;
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
