// Sparse flash attention over the paged int8 latent-KV cache, gfx950 (MI355X).
//
// Semantics: sparse_flash_attention_quant_compute of the reference example
// (examples/models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:106-207) with the
// online-softmax numerics of its flash variant (same file :271-417): per query row the first
// cur_seq entries of the top-k index row are translated through the block table, the int8 latent
// rows are de-quantised to bf16 (bf16_rne(float(int8) * scale[c / 128])), scores are bf16 x bf16
// products accumulated in fp32 over 576 dims, softmax runs in fp32, P is rounded to bf16
// un-normalised, PV accumulates in fp32 over 512 dims and the result is divided by the fp32 row sum.
//
// Work decomposition: one workgroup = (query row, group of 32*NW heads, key split).  Each of the NW
// waves owns 32 heads for both matrix products, so probabilities never leave registers:
//   S^T[key][head] = K[key][:] . Q^T        v_mfma_f32_32x32x16_bf16, A = K tile rows from LDS,
//                                            B = Q^T fragments resident in registers
//   O^T[dv][head] += V^T[dv][key] . P^T     A = V^T read from the same LDS tile with the
//                                            transposing LDS read, B = P^T straight from the
//                                            accumulator registers of the first product
// (the accumulator layout of a 32x32 product gives lane (head, half) the keys 8*(r/4)+4*half+r%4;
// the transposed V read uses the same key order, so no cross-lane movement is needed).
// All NW waves gather and de-quantise the tile cooperatively: each selected row is read once per
// workgroup (512 B int8 + 128 B rope + 16 B scales) and written to LDS as 576 bf16.
#include "common.h"
#include "sfa_kernels.h"

namespace pto {
namespace {

constexpr int DN = 512;           // latent (nope) width = value width
constexpr int DR = 64;            // rope width
constexpr int D = DN + DR;        // score contraction width
constexpr int KT = 32;            // keys per tile
constexpr int PITCH = D + 8;      // LDS row pitch in bf16 elements (1168 B: rows land 4 banks apart)
constexpr int KSTEPS = D / 16;    // 36 contraction steps of 16
constexpr int DVB = DN / 32;      // 16 output blocks of 32 value channels

// 16 int8 (one 16-byte load) times one scale -> 16 bf16 as two 16-byte LDS stores
__device__ __forceinline__ void dequant16(const i32x4 raw, const float sc, uint16_t *dst)
{
    u32x4 lo, hi;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const int v = raw[w];
        const float f0 = (float)((v << 24) >> 24) * sc;
        const float f1 = (float)((v << 16) >> 24) * sc;
        const float f2 = (float)((v << 8) >> 24) * sc;
        const float f3 = (float)(v >> 24) * sc;
        const uint32_t p0 = pack_bf16x2(f0, f1);
        const uint32_t p1 = pack_bf16x2(f2, f3);
        if (w < 2) { lo[2 * w] = p0; lo[2 * w + 1] = p1; }
        else { hi[2 * (w - 2)] = p0; hi[2 * (w - 2) + 1] = p1; }
    }
    *reinterpret_cast<u32x4 *>(dst) = lo;
    *reinterpret_cast<u32x4 *>(dst + 8) = hi;
}

// O^T accumulators live in the accumulation registers for the whole kernel (16 blocks x 16 = all 256 of
// them).  Every instruction that touches them inside the key loop is inline assembly with an
// accumulation-register constraint, so the register allocator cannot migrate them into the 256
// architectural registers, most of which hold the Q^T fragments.
__device__ __forceinline__ void acc_mfma(f32x16 &acc, const bf16x8 a, const bf16x8 b)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// acc *= alpha, one register at a time through a single architectural temporary (rare path)
__device__ __forceinline__ void acc_scale(f32x16 &acc, const float alpha)
{
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        float e = acc[r];
        float tmp;
        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %2, %1\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                     : "+a"(e), "=&v"(tmp)
                     : "v"(alpha));
        acc[r] = e;
    }
}

template <int I, int N> struct AccLoop {
    static __device__ __forceinline__ void scale(f32x16 *o, float a) { acc_scale(o[I], a); AccLoop<I + 1, N>::scale(o, a); }
    static __device__ __forceinline__ void pv(f32x16 *o, const uint16_t *v, const bf16x8 pf)
    {
        const s16x4 lo = lds_read_tr16(v + 32 * I);
        const s16x4 hi = lds_read_tr16(v + 32 * I + 8 * PITCH);
        const s16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc_mfma(o[I], __builtin_bit_cast(bf16x8, a), pf);
        if ((I & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // bound how many V^T reads are hoisted
        AccLoop<I + 1, N>::pv(o, v, pf);
    }
};
template <int N> struct AccLoop<N, N> {
    static __device__ __forceinline__ void scale(f32x16 *, float) {}
    static __device__ __forceinline__ void pv(f32x16 *, const uint16_t *, const bf16x8) {}
};

// Wait states the hardware does not interlock: a matrix-core write followed by a vector-ALU read of
// the same register needs up to 19 idle issue slots.
__device__ __forceinline__ void mfma_to_valu_fence() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
__device__ __forceinline__ void valu_to_mfma_fence() { asm volatile("s_nop 4" ::: "memory"); }

constexpr float RESCALE_TAU = 8.0f;   // log2 units: the reference max moves only when exceeded by 2^8

template <int NW>
__global__ __launch_bounds__(NW * 64) void sfa_decode_kernel(const SfaParams p)
{
    __shared__ __attribute__((aligned(16))) uint16_t tile[KT * PITCH];
    __shared__ int rows_lds[SFA_MAX_CHUNK];

    const int tid = threadIdx.x;
    const int w = tid >> 6;
    const int l = tid & 63;
    const int half = l >> 5;
    const int col = l & 31;

    // workgroups of one query row share an XCD (consecutive workgroup ids rotate over the 8 XCDs)
    const int per_row = p.hgroups * p.nsplit;
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int t = (slot / per_row) * 8 + xcd;
    if (t >= p.T) return;
    const int within = slot % per_row;
    const int hg = within / p.nsplit;
    const int sp = within % p.nsplit;
    const int b = t / p.S1;
    const int s1i = t - b * p.S1;

    int cur = p.act[b] - p.S1 + 1 + s1i;
    cur = cur < 0 ? 0 : (cur > p.topk ? p.topk : cur);
    const int ntile = (cur + KT - 1) / KT;
    const int tiles_per_split = (ntile + p.nsplit - 1) / p.nsplit;
    const int k_begin = sp * tiles_per_split * KT;
    int k_end = k_begin + tiles_per_split * KT;
    k_end = k_end > cur ? cur : k_end;

    const int head = hg * (32 * NW) + w * 32 + col;
    const bool head_ok = head < p.NQ;

    // logical position -> physical cache row for this split's keys
    for (int i = tid; i < k_end - k_begin; i += NW * 64) {
        const int idx = p.topk_idx[(size_t)t * p.topk + k_begin + i];
        int blk = idx / p.bs;
        blk = blk < 0 ? 0 : (blk >= p.maxblk ? p.maxblk - 1 : blk);
        long long row = (long long)p.bt[(size_t)b * p.maxblk + blk] * p.bs + (idx - (idx / p.bs) * p.bs);
        row = row < 0 ? 0 : (row >= p.kv_rows ? p.kv_rows - 1 : row);
        rows_lds[i] = (int)row;
    }

    // Q^T fragments: lane (head, half) holds q[head][16*ks + 8*half .. +8]; lanes of heads past NQ
    // compute on row 0 of the query and are never stored
    bf16x8 qf[KSTEPS];
    {
        const size_t qrow = (size_t)t * p.NQ + (head_ok ? head : 0);
        const uint16_t *qn = p.q_nope + qrow * DN + 8 * half;
        const uint16_t *qr = p.q_rope + qrow * DR + 8 * half;
#pragma unroll
        for (int ks = 0; ks < DN / 16; ++ks) qf[ks] = *reinterpret_cast<const bf16x8 *>(qn + 16 * ks);
#pragma unroll
        for (int ks = 0; ks < DR / 16; ++ks) qf[DN / 16 + ks] = *reinterpret_cast<const bf16x8 *>(qr + 16 * ks);
    }

    f32x16 o[DVB];
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    valu_to_mfma_fence();
    float m_run = -INFINITY;   // reference max, log2 domain
    float l_run = 0.f;         // running sum of exp2(s - m_run)

    __syncthreads();

    for (int kt = k_begin; kt < k_end; kt += KT) {
        // ---- gather + de-quantise KT rows into LDS (each wave KT/NW rows, two rows per pass)
#pragma unroll
        for (int i = 0; i < KT / (2 * NW); ++i) {
            const int kl = w * (KT / NW) + 2 * i + half;
            const bool valid = kt + kl < k_end;
            const int row = valid ? rows_lds[kt - k_begin + kl] : 0;
            i32x4 raw = {0, 0, 0, 0};
            float sc = 0.f;
            if (valid) {
                raw = *reinterpret_cast<const i32x4 *>(p.kn + (size_t)row * DN + 16 * col);
                sc = p.ksc[(size_t)row * 4 + (col >> 3)];
            }
            dequant16(raw, sc, tile + kl * PITCH + 16 * col);
        }
        for (int i = tid; i < KT * (DR / 8); i += NW * 64) {
            const int kl = i >> 3;
            const int part = i & 7;
            const bool valid = kt + kl < k_end;
            u32x4 v = {0, 0, 0, 0};
            if (valid) {
                const int row = rows_lds[kt - k_begin + kl];
                v = *reinterpret_cast<const u32x4 *>(p.kr + (size_t)row * DR + 8 * part);
            }
            *reinterpret_cast<u32x4 *>(tile + kl * PITCH + DN + 8 * part) = v;
        }
        __syncthreads();

        // ---- S^T = K . Q^T
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        {
            const uint16_t *arow = tile + col * PITCH + 8 * half;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(arow + 16 * ks);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s, 0, 0, 0);
                if ((ks & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- online softmax; lane (head, half) holds keys kt + 8*(r/4) + 4*half + r%4
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kt + 8 * (r >> 2) + 4 * half + (r & 3);
            s[r] = key < k_end ? s[r] * p.scale_log2 : -INFINITY;
            mx = fmaxf(mx, s[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // The reference max follows the true max lazily: probabilities may reach 2^RESCALE_TAU, which
        // fp32 sums and bf16 P hold without loss, and the accumulators are rescaled only on a jump.
        const bool upd = mx > m_run + RESCALE_TAU;          // always true on the first tile (m_run = -inf)
        const float m_new = upd ? mx : m_run;
        const float alpha = upd ? exp2f(m_run - m_new) : 1.0f;
        const bool rescale = upd && l_run > 0.f;            // nothing accumulated yet: nothing to rescale
        float lsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] = exp2f(s[r] - m_new);
            lsum += s[r];
        }
        lsum += __shfl_xor(lsum, 32);
        l_run = l_run * alpha + lsum;
        m_run = m_new;
        if (__any(rescale)) {
            mfma_to_valu_fence();
            AccLoop<0, DVB>::scale(o, alpha);
            valu_to_mfma_fence();
        }
        bf16x8 pf[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            u32x4 pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = pack_bf16x2(s[8 * kk + 2 * e], s[8 * kk + 2 * e + 1]);
            pf[kk] = __builtin_bit_cast(bf16x8, pk);
        }

        // ---- O^T += V^T . P^T
        {
            const uint16_t *vbase = tile + (4 * half + ((l & 15) >> 2)) * PITCH + 16 * ((l >> 4) & 1) + 4 * (l & 3);
            AccLoop<0, DVB>::pv(o, vbase, pf[0]);
            AccLoop<0, DVB>::pv(o, vbase + 16 * PITCH, pf[1]);
        }
        __syncthreads();
    }

    // ---- epilogue: lane (head, half) holds value channels 32*dvb + 8*(r/4) + 4*half + r%4
    if (!head_ok) return;
    mfma_to_valu_fence();
    if (p.nsplit == 1) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        uint16_t *orow = p.out + ((size_t)t * p.NQ + head) * DN + 4 * half;
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                u32x2 v;
                v[0] = pack_bf16x2(o[dvb][4 * q4] * inv, o[dvb][4 * q4 + 1] * inv);
                v[1] = pack_bf16x2(o[dvb][4 * q4 + 2] * inv, o[dvb][4 * q4 + 3] * inv);
                *reinterpret_cast<u32x2 *>(orow + 32 * dvb + 8 * q4) = v;
            }
    } else {
        const size_t prow = ((size_t)t * p.nsplit + sp) * p.NQ + head;
        float *po = p.part_o + prow * DN + 4 * half;
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                f32x4 v = {o[dvb][4 * q4], o[dvb][4 * q4 + 1], o[dvb][4 * q4 + 2], o[dvb][4 * q4 + 3]};
                *reinterpret_cast<f32x4 *>(po + 32 * dvb + 8 * q4) = v;
            }
        if (half == 0) {
            p.part_ml[prow * 2] = m_run;
            p.part_ml[prow * 2 + 1] = l_run;
        }
    }
}

// Merges the key splits of one query row: out = sum_s 2^(m_s - m) acc_s / sum_s 2^(m_s - m) l_s.
// One thread per (row, head, 4 value channels).
__global__ __launch_bounds__(256) void sfa_combine_kernel(const SfaParams p)
{
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)p.T * p.NQ * (DN / 4);
    if (gid >= total) return;
    const int c4 = (int)(gid % (DN / 4));
    const size_t th = gid / (DN / 4);
    const int head = (int)(th % p.NQ);
    const int t = (int)(th / p.NQ);
    float m = -INFINITY;
    for (int s = 0; s < p.nsplit; ++s) {
        const size_t prow = ((size_t)t * p.nsplit + s) * p.NQ + head;
        m = fmaxf(m, p.part_ml[prow * 2]);
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float lsum = 0.f;
    for (int s = 0; s < p.nsplit; ++s) {
        const size_t prow = ((size_t)t * p.nsplit + s) * p.NQ + head;
        const float ms = p.part_ml[prow * 2];
        const float ls = p.part_ml[prow * 2 + 1];
        if (ls > 0.f) {
            const float wgt = exp2f(ms - m);
            const f32x4 v = *reinterpret_cast<const f32x4 *>(p.part_o + prow * DN + 4 * c4);
            acc += v * wgt;
            lsum += ls * wgt;
        }
    }
    const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
    u32x2 v;
    v[0] = pack_bf16x2(acc[0] * inv, acc[1] * inv);
    v[1] = pack_bf16x2(acc[2] * inv, acc[3] * inv);
    *reinterpret_cast<u32x2 *>(p.out + ((size_t)t * p.NQ + head) * DN + 4 * c4) = v;
}

}  // namespace

hipError_t sfa_launch(const SfaParams &p, hipStream_t stream)
{
    const int rows8 = (p.T + 7) / 8 * 8;
    const unsigned grid = (unsigned)(rows8 * p.hgroups * p.nsplit);
    switch (p.waves) {
    case 1: hipLaunchKernelGGL(sfa_decode_kernel<1>, dim3(grid), dim3(64), 0, stream, p); break;
    case 2: hipLaunchKernelGGL(sfa_decode_kernel<2>, dim3(grid), dim3(128), 0, stream, p); break;
    default: hipLaunchKernelGGL(sfa_decode_kernel<4>, dim3(grid), dim3(256), 0, stream, p); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.nsplit > 1) {
        const size_t total = (size_t)p.T * p.NQ * (DN / 4);
        hipLaunchKernelGGL(sfa_combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace pto
