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
//   li_wscale_kernel  w_scale[t,h] = fp16(q_scale * weight) if both fp16, else the fp32 product
//   li_score_kernel   one wave per run of 32-key blocks: v_mfma_i32_32x32x32_i8 with A = the
//                     token's 64 query heads (two 32-row operands resident in registers) and
//                     B = 32 key rows loaded straight from the paged cache in operand layout;
//                     epilogue in registers; scores to a [T, max_seq] fp32 workspace
//   li_select_kernel  one workgroup per query token: 4-pass radix select (8 bits per pass) on an
//                     order-preserving 32-bit image of the score, deterministic compaction in
//                     position order, bitonic sort of the survivors by (score desc, position asc)
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

constexpr int BPW = 8;                       // 32-key blocks per wave
constexpr int WG_KEYS = 4 * BPW * 32;        // keys per 256-thread workgroup

__device__ __forceinline__ float load_scalar(const void *p, size_t i, int dt)
{
    if (dt == PTO_DT_FP32) return static_cast<const float *>(p)[i];
    const uint16_t h = static_cast<const uint16_t *>(p)[i];
    if (dt == PTO_DT_BF16) return bf16_bits_to_f32(h);
    return (float)__builtin_bit_cast(_Float16, h);
}

__global__ __launch_bounds__(256) void li_wscale_kernel(const LiParams p)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= p.T * LI_HEADS) return;
    const float qs = load_scalar(p.q_scale, i, p.q_dt);
    const float w = load_scalar(p.weight, i, p.w_dt);
    float prod = __fmul_rn(qs, w);
    if (p.q_dt == PTO_DT_FP16 && p.w_dt == PTO_DT_FP16) prod = (float)(_Float16)prod;   // fp16 x fp16 -> fp16
    p.w_scale[i] = prod;
}

// relu, scale by 2^-11, round to fp16, back to fp32
__device__ __forceinline__ float relu_fp16_term(const int dot)
{
    const float r = (float)(dot > 0 ? dot : 0) * (1.0f / 2048.0f);
    return (float)(_Float16)r;
}

__global__ __launch_bounds__(256) void li_score_kernel(const LiParams p)
{
    const int t = blockIdx.y;
    const int b = t / p.S1;
    int cur = p.act[b];
    const int cap = p.maxblk * p.bs;
    cur = cur < 0 ? 0 : (cur > cap ? cap : cur);
    const int w = threadIdx.x >> 6;
    const int l = threadIdx.x & 63;
    const int j = l & 31;
    const int half = l >> 5;
    const int key0 = blockIdx.x * WG_KEYS + w * (BPW * 32);
    if (key0 >= cur) return;

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
    float wsc[32];
#pragma unroll
    for (int r = 0; r < 32; ++r) wsc[r] = p.w_scale[(size_t)t * LI_HEADS + 32 * half + r];

    float *srow = p.scores + (size_t)t * p.score_stride;
    for (int blk = 0; blk < BPW; ++blk) {
        const int pos0 = key0 + 32 * blk;
        if (pos0 >= cur) break;
        const int page = pos0 / p.bs;
        int pb = p.bt[(size_t)b * p.maxblk + page];
        pb = pb < 0 ? 0 : (pb >= p.nblocks ? p.nblocks - 1 : pb);
        const size_t row = (size_t)pb * p.bs + (pos0 - page * p.bs) + j;
        const int8_t *kp = p.kcache + row * LI_DIM + 64 * half;
        i32x4 kf[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) kf[ks] = *reinterpret_cast<const i32x4 *>(kp + 16 * ks);
        const float ksc = load_scalar(p.k_scale, row, p.k_dt);

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
        if (half == 1 && pos0 + j < cur) srow[pos0 + j] = __fmul_rn(hi, ksc);
    }
}

// ---------------------------------------------------------------------------------- select

constexpr int SEL_THREADS = 1024;
constexpr int SEL_WAVES = SEL_THREADS / 64;

// order-preserving image of a score: larger score <=> larger key; -0.0 and +0.0 map to one key
__device__ __forceinline__ uint32_t score_key(const float x)
{
    uint32_t u = __float_as_uint(x);
    u = u == 0x80000000u ? 0u : u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(SEL_THREADS) void li_select_kernel(const LiParams p)
{
    __shared__ uint32_t hist[256];
    __shared__ unsigned long long sortbuf[LI_MAX_SELECT];
    __shared__ uint32_t wave_gt[SEL_WAVES], wave_eq[SEL_WAVES];
    __shared__ uint32_t sh_prefix, sh_krem;

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

}  // namespace

hipError_t li_launch(const LiParams &p, hipStream_t stream)
{
    hipLaunchKernelGGL(li_wscale_kernel, dim3((unsigned)((p.T * LI_HEADS + 255) / 256)), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const unsigned gx = (unsigned)((p.score_stride + WG_KEYS - 1) / WG_KEYS);
    hipLaunchKernelGGL(li_score_kernel, dim3(gx, (unsigned)p.T), dim3(256), 0, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(li_select_kernel, dim3((unsigned)p.T), dim3(SEL_THREADS), 0, stream, p);
    return hipGetLastError();
}

}  // namespace pto
