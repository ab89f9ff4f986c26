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
// workgroup (512 B int8 + 128 B rope + 16 B scales, from three arrays or from one packed 656-byte row)
// and written to LDS as 576 bf16.
#include <type_traits>

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

// 8 int8 (two dwords of a 16-byte load) times one scale -> 8 bf16 as one 16-byte LDS store.
// x*sc is formed as fma(float(x + 128), sc, -128*sc): the byte is biased to unsigned so that a single
// v_cvt_f32_ubyteN converts it, and the fused multiply-add rounds the exact product (x*sc) once, which
// is bit-identical to the rounded multiply (128*sc is exact).
__device__ __forceinline__ void dequant8(const int r0, const int r1, const float sc, uint16_t *dst)
{
    const float bias = -128.0f * sc;
    u32x4 out;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        const uint32_t v = (uint32_t)(w == 0 ? r0 : r1) ^ 0x80808080u;
        const float f0 = __builtin_fmaf((float)(v & 0xffu), sc, bias);
        const float f1 = __builtin_fmaf((float)((v >> 8) & 0xffu), sc, bias);
        const float f2 = __builtin_fmaf((float)((v >> 16) & 0xffu), sc, bias);
        const float f3 = __builtin_fmaf((float)(v >> 24), sc, bias);
        out[2 * w] = pack_bf16x2(f0, f1);
        out[2 * w + 1] = pack_bf16x2(f2, f3);
    }
    *reinterpret_cast<u32x4 *>(dst) = out;
}

// O^T accumulators live in the accumulation registers for the whole kernel (16 blocks x 16 = all 256 of
// them).  Inside the key loop they are touched only by the matrix product itself and by acc_scale,
// which works on them in place through inline assembly: any plain C++ arithmetic on them makes the
// register allocator migrate them into the 256 architectural registers, most of which hold the Q^T
// fragments (observed: hundreds of spilled registers).
__device__ __forceinline__ void acc_mfma(f32x16 &acc, const bf16x8 a, const bf16x8 b)
{
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
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
};
template <int N> struct AccLoop<N, N> {
    static __device__ __forceinline__ void scale(f32x16 *, float) {}
};

// Wait states the hardware does not interlock: a matrix-core write followed by a vector-ALU read of
// the same register needs up to 19 idle issue slots.
__device__ __forceinline__ void mfma_to_valu_fence() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
__device__ __forceinline__ void valu_to_mfma_fence() { asm volatile("s_nop 4" ::: "memory"); }

constexpr float RESCALE_TAU = 8.0f;   // log2 units: the reference max moves only when exceeded by 2^8

// QUANT: the latent part of a cache row is int8 with four fp32 scales and is de-quantised on the way into
// LDS; otherwise it is bf16 already (1024 bytes) and travels cache -> LDS tile directly by LDS-DMA.
template <int NW, bool QUANT>
__global__ __launch_bounds__(NW * 64) void sfa_decode_kernel(const SfaParams p)
{
    // One LDS pool.  Prologue: all 32*NW query heads staged at once (PITCH elements each).  Loop: tile
    // buffers of KT rows -- while tile n is consumed from one, tile n+1 (loaded into registers before
    // the matrix products of tile n were issued) is de-quantised into the other; one barrier per tile.
    // Epilogue: per-wave transposition slices.
    constexpr int POOL_ROWS = 32 * NW > 2 * KT ? 32 * NW : 2 * KT;     // at least the two tile buffers
    __shared__ __attribute__((aligned(16))) uint16_t pool[POOL_ROWS * PITCH];
    __shared__ int rows_lds[SFA_MAX_CHUNK + KT];
    uint16_t *const tile0 = pool;
    uint16_t *const tile1 = pool + KT * PITCH;

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

    // Q^T fragments: lane (head, half) holds q[head][16*ks + 8*half .. +8].  Read straight from global
    // memory each such load would touch 32 rows; instead every wave stages its own 32 heads in its slice
    // of the LDS pool with LDS-DMA requests of whole cache lines, in two passes: nope chunks 0..31 of
    // every head, then nope chunks 32..63 plus the 8 rope chunks (a chunk is 16 bytes).  A nope request
    // covers two heads (lane = 32*(head & 1) + position), a rope request eight (lane = 8*(head & 7) +
    // position); position pos of head h holds chunk pos ^ (h & 7), which makes the fragment reads
    // conflict-free.  The cache address is a wave-uniform base plus a per-lane offset.  Heads past NQ
    // read the last head and are never stored.  The second pass stays in flight while the row table
    // below is built.
    bf16x8 qf[KSTEPS];
    constexpr int QREGION = 20 * 1024;                            // per wave: 16 KiB nope half + 4 KiB rope
    static_assert(NW * QREGION <= POOL_ROWS * PITCH * 2, "Q staging must fit in the pool");
    uint8_t *const qreg = reinterpret_cast<uint8_t *>(pool) + w * QREGION;
    const uint32_t qdst = (uint32_t)(uintptr_t)(lds_byte_t *)qreg;
    const int q_head0 = hg * (32 * NW) + w * 32;
    auto request_q = [&](const int pass) {
        if (q_head0 + 32 <= p.NQ) {                               // wave-uniform: all 32 heads exist
            const size_t qrow0 = (size_t)t * p.NQ + q_head0;
#pragma unroll 1
            for (int i = 0; i < 16; ++i) {
                const int h = 2 * i + half;
                const uint32_t off = (uint32_t)(half * (DN * 2) + (((pass * 32) + (col ^ (h & 7))) << 4));
                dma16_base(p.q_nope + (qrow0 + 2 * i) * DN, off, qdst + i * 1024);
            }
            if (pass == 1) {
                const uint32_t off = (uint32_t)((l >> 3) * (DR * 2) + (((l & 7) ^ (l >> 3)) << 4));
#pragma unroll 1
                for (int j = 0; j < 4; ++j) dma16_base(p.q_rope + (qrow0 + 8 * j) * DR, off, qdst + 16 * 1024 + j * 1024);
            }
        } else {
#pragma unroll 1
            for (int i = 0; i < 16; ++i) {
                const int h = 2 * i + half;
                int hd = q_head0 + h;
                hd = hd < p.NQ ? hd : p.NQ - 1;
                dma16(p.q_nope + ((size_t)t * p.NQ + hd) * DN + 8 * ((pass * 32) + (col ^ (h & 7))), qdst + i * 1024);
            }
            if (pass == 1) {
#pragma unroll 1
                for (int j = 0; j < 4; ++j) {
                    const int h = 8 * j + (l >> 3);
                    int hd = q_head0 + h;
                    hd = hd < p.NQ ? hd : p.NQ - 1;
                    dma16(p.q_rope + ((size_t)t * p.NQ + hd) * DR + 8 * ((l & 7) ^ (l >> 3)), qdst + 16 * 1024 + j * 1024);
                }
            }
        }
    };
    auto collect_q = [&](const int pass) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                       // vmcnt(0): the pass has landed
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 16; ++ks)
            qf[16 * pass + ks] = *reinterpret_cast<const bf16x8 *>(qreg + col * 512 + (((2 * ks + half) ^ (col & 7)) << 4));
        if (pass == 1) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
                qf[32 + ks] = *reinterpret_cast<const bf16x8 *>(qreg + 16 * 1024 + col * 128 + (((2 * ks + half) ^ (col & 7)) << 4));
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);                       // lgkmcnt(0): the slice may be overwritten
    };
    request_q(0);
    collect_q(0);
    request_q(1);

    // logical position -> physical cache row for this split's keys.  The table is padded to a whole
    // number of tiles plus one with the row of the split's first key: keys past k_end are then loaded
    // like any other (finite data) and masked out of the softmax, and the loop can prefetch "the next
    // tile" unconditionally -- no per-key and no per-tile branches.
    {
        const int n_valid = k_end - k_begin;
        const int n_pad = n_valid > 0 ? (n_valid + KT - 1) / KT * KT + KT : 0;   // + one tile: see the loop
        for (int i = tid; i < n_pad; i += NW * 64) {
            const int idx = p.topk_idx[(size_t)t * p.topk + k_begin + (i < n_valid ? i : 0)];
            int blk = idx / p.bs;
            blk = blk < 0 ? 0 : (blk >= p.maxblk ? p.maxblk - 1 : blk);
            long long row = (long long)p.bt[(size_t)b * p.maxblk + blk] * p.bs + (idx - (idx / p.bs) * p.bs);
            row = row < 0 ? 0 : (row >= p.kv_rows ? p.kv_rows - 1 : row);
            rows_lds[i] = (int)row;
        }
    }

    f32x16 o[DVB];
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    valu_to_mfma_fence();
    float m_run = -INFINITY;   // reference max, log2 domain
    float l_run = 0.f;         // running sum of exp2(s - m_run)

    // gather registers of one tile: NP passes of two keys per wave (512 B int8 each), RP rope pieces
    constexpr int NP = KT / (2 * NW);
    constexpr int RP = (KT * (DR / 8)) / (NW * 64);
    i32x4 raw[NP];
    float rsc[NP];
    u32x4 rrope[RP];

    // wave w gathers keys w*KT/NW .. +KT/NW of the tile; within a pass the lower half-wave takes key
    // half*NP + i, so a lane's NP row numbers are one contiguous LDS read
    auto issue_loads = [&](const int kt, uint16_t *buf) {
        if (QUANT) {
            const int *rtab = rows_lds + (kt - k_begin) + w * (KT / NW) + half * NP;
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int row = rtab[i];
                raw[i] = *reinterpret_cast<const i32x4 *>(p.kn + (size_t)row * p.kn_pitch + 16 * col);
                rsc[i] = *reinterpret_cast<const float *>(p.ksc + (size_t)row * p.ksc_pitch + 4 * (col >> 3));
            }
        } else {
            // one request per key: the 64 lanes' 16-byte pieces are the 1024 bytes of the row, in order
            const int *rtab = rows_lds + (kt - k_begin) + w * (KT / NW);
#pragma unroll
            for (int i = 0; i < KT / NW; ++i)
                dma16(p.kn + (size_t)rtab[i] * p.kn_pitch + 16 * l,
                      (uint32_t)(uintptr_t)(lds_byte_t *)(buf + (w * (KT / NW) + i) * PITCH));
        }
#pragma unroll
        for (int i = 0; i < RP; ++i) {
            const int e = tid + i * NW * 64;
            const int row = rows_lds[(kt - k_begin) + (e >> 3)];
            rrope[i] = *reinterpret_cast<const u32x4 *>(p.kr + (size_t)row * p.kr_pitch + 16 * (e & 7));
        }
    };
    // de-quantise and store one eighth of the gathered tile (piece 0 also stores the rope part)
    auto store_piece = [&](uint16_t *buf, const int piece) {
        static_assert(NP * 2 % 8 == 0 || NP * 2 == 8 || true, "");
        constexpr int HALVES = 2 * NP;                 // 16-byte LDS stores of this lane per tile
        constexpr int PER = (HALVES + 7) / 8;          // ... per piece
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int hidx = piece * PER + q;
            if (QUANT && hidx < HALVES) {
                const int i = hidx >> 1, hh = hidx & 1;
                const int kl = w * (KT / NW) + half * NP + i;
                dequant8(raw[i][2 * hh], raw[i][2 * hh + 1], rsc[i], buf + kl * PITCH + 16 * col + 8 * hh);
            }
        }
        if (piece == 0) {
#pragma unroll
            for (int i = 0; i < RP; ++i) {
                const int e = tid + i * NW * 64;
                *reinterpret_cast<u32x4 *>(buf + (e >> 3) * PITCH + DN + 8 * (e & 7)) = rrope[i];
            }
        }
    };
    auto store_tile = [&](uint16_t *buf) {
#pragma unroll
        for (int piece = 0; piece < 8; ++piece) store_piece(buf, piece);
    };

    collect_q(1);
    __syncthreads();                       // row table complete, pool free again
    if (k_begin < k_end) {
        issue_loads(k_begin, tile0);
        store_tile(tile0);
    }
    if (!QUANT) __builtin_amdgcn_s_waitcnt(0x0F70);     // this wave's direct requests into the tile have landed
    __syncthreads();
    // All global loads issued so far (Q^T fragments, first tile) are complete from here on, so that
    // inside the loop the only outstanding vector-memory operations are the next tile's gather and
    // the compiler's wait counts do not serialise it with the matrix products.
    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0), expcnt and lgkmcnt unconstrained

    int it = 0;
    for (int kt = k_begin; kt < k_end; kt += KT, ++it) {
        const uint16_t *cur_tile = (it & 1) ? tile1 : tile0;
        uint16_t *nxt_tile = (it & 1) ? tile0 : tile1;
        issue_loads(kt + KT, nxt_tile);          // next tile (or the padding tile): in flight during the products

        // ---- S^T = K . Q^T, LDS reads running one group of four contraction steps ahead
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        {
            const uint16_t *arow = cur_tile + col * PITCH + 8 * half;
            bf16x8 fa[2][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) fa[0][e] = *reinterpret_cast<const bf16x8 *>(arow + 16 * e);
#pragma unroll
            for (int g = 0; g < KSTEPS / 4; ++g) {
                if (g + 1 < KSTEPS / 4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        fa[(g + 1) & 1][e] = *reinterpret_cast<const bf16x8 *>(arow + 16 * (4 * (g + 1) + e));
                }
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[g & 1][e], qf[4 * g + e], s, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- online softmax; lane (head, half) holds keys kt + 8*(r/4) + 4*half + r%4
        float mx = -INFINITY;
        if (kt + KT > k_end) {                  // only the split's last tile can hold keys past k_end
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (kt + 8 * (r >> 2) + 4 * half + (r & 3) >= k_end) s[r] = -INFINITY;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] *= p.scale_log2;
            mx = fmaxf(mx, s[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // The reference max follows the true max lazily: probabilities may reach 2^RESCALE_TAU, which
        // fp32 sums and bf16 P hold without loss, and the accumulators are rescaled only on a jump.
        const bool upd = mx > m_run + RESCALE_TAU;          // always true on the first tile (m_run = -inf)
        const float m_new = upd ? mx : m_run;
        const float alpha = upd ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
        const bool rescale = upd && l_run > 0.f;            // nothing accumulated yet: nothing to rescale
        float lsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] = __builtin_amdgcn_exp2f(s[r] - m_new);      // v_exp_f32; exp2(-inf) = 0
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

        // ---- O^T += V^T . P^T: product m = 16*kk + dvb, V^T reads one group of four products ahead;
        // interleaved with the de-quantisation of the next tile into the other buffer
        {
            const uint16_t *vbase = cur_tile + (4 * half + ((l & 15) >> 2)) * PITCH + 16 * ((l >> 4) & 1) + 4 * (l & 3);
            s16x4 va[2][4][2];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                va[0][e][0] = lds_read_tr16(vbase + 32 * e);
                va[0][e][1] = lds_read_tr16(vbase + 32 * e + 8 * PITCH);
            }
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g + 1 < 8) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int m = 4 * (g + 1) + e;
                        const uint16_t *a0 = vbase + (16 * (m >> 4)) * PITCH + 32 * (m & 15);
                        va[(g + 1) & 1][e][0] = lds_read_tr16(a0);
                        va[(g + 1) & 1][e][1] = lds_read_tr16(a0 + 8 * PITCH);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = 4 * g + e;
                    const s16x8 a = __builtin_shufflevector(va[g & 1][e][0], va[g & 1][e][1], 0, 1, 2, 3, 4, 5, 6, 7);
                    acc_mfma(o[m & 15], __builtin_bit_cast(bf16x8, a), pf[m >> 4]);
                }
                // one eighth of the next tile's de-quantisation rides in the shadow of these products
                store_piece(nxt_tile, g);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (!QUANT) __builtin_amdgcn_s_waitcnt(0x0F70); // this wave's direct requests into the next tile have landed
        __syncthreads();
    }

    // ---- epilogue.  Lane (head, half) holds value channels 32*dvb + 8*(r/4) + 4*half + r%4 of its head;
    // written from there each store instruction would touch 32 rows with 32 bytes each.  Each wave
    // instead transposes 128 channels at a time through its own slice of the (now idle) tile
    // memory, so that 32 lanes write 512 contiguous bytes of one head (256 for the bf16 result).
    mfma_to_valu_fence();
    {
        // staging slice of this wave: 32 heads x 128 channels fp32, 16-byte chunk c of head h stored at
        // chunk c ^ (h & 7): both the column-wise writes and the row-wise reads are bank-conflict free.
        // The accumulators go to LDS as they are (the 1/l factor is applied on the way out, from a
        // small per-head table), and the way out is a rolled loop: the straight-line part of the
        // epilogue is one LDS store per four accumulator registers.
        float *stage = reinterpret_cast<float *>(pool) + w * (32 * 128);
        float *inv_tab = reinterpret_cast<float *>(rows_lds) + w * 32;      // the row table is dead by now
        const int head_base = hg * (32 * NW) + w * 32;
        const size_t prow_base = ((size_t)t * p.nsplit + sp) * p.NQ;
        if (half == 0) inv_tab[col] = l_run > 0.f ? 1.0f / l_run : 0.f;
        // FINAL: bf16 result rows; otherwise fp16 partial of a key split (O / l of the split, merged by
        // the combine kernel with weights l * 2^(m - m_max); O / l is a convex combination of
        // de-quantised V rows, so it stays finite in fp16 as long as |int8 * scale| < 65504).
        // ALL: every head of this wave exists, so the stores need no predicate.  Both are uniform
        // and resolved outside the loops: scalar branches inside them cost more than the work.
        auto drain = [&](auto final_tag, auto all_tag) {
            constexpr bool FINAL = decltype(final_tag)::value;
            constexpr bool ALL = decltype(all_tag)::value;
            uint16_t *dst0 = FINAL ? p.out + ((size_t)t * p.NQ + head_base + half) * DN + 4 * col
                                   : p.part_o + (prow_base + head_base + half) * DN + 4 * col;
#pragma unroll
            for (int gq = 0; gq < DVB / 4; ++gq) {
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        const f32x16 &acc = o[4 * gq + b4];
                        const f32x4 v = {acc[4 * q4], acc[4 * q4 + 1], acc[4 * q4 + 2], acc[4 * q4 + 3]};
                        *reinterpret_cast<f32x4 *>(stage + col * 128 + 4 * ((8 * b4 + 2 * q4 + half) ^ (col & 7))) = v;
                    }
#pragma unroll 1
                for (int pq = 0; pq < 2; ++pq) {
                    f32x4 rv[8];
                    float iv[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int hl = 2 * (8 * pq + e) + half;
                        rv[e] = *reinterpret_cast<const f32x4 *>(stage + hl * 128 + 4 * (col ^ (hl & 7)));
                        iv[e] = inv_tab[hl];
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int hl = 2 * (8 * pq + e) + half;
                        const f32x4 v = rv[e] * iv[e];
                        u32x2 pk;
                        pk[0] = FINAL ? pack_bf16x2(v[0], v[1]) : pack_f16x2(v[0], v[1]);
                        pk[1] = FINAL ? pack_bf16x2(v[2], v[3]) : pack_f16x2(v[2], v[3]);
                        if (ALL || head_base + hl < p.NQ)
                            *reinterpret_cast<u32x2 *>(dst0 + (size_t)(hl - half) * DN + 128 * gq) = pk;
                    }
                }
            }
        };
        const bool all_heads = head_base + 32 <= p.NQ;
        if (p.nsplit == 1) {
            if (all_heads) drain(std::true_type{}, std::true_type{});
            else drain(std::true_type{}, std::false_type{});
        } else {
            if (all_heads) drain(std::false_type{}, std::true_type{});
            else drain(std::false_type{}, std::false_type{});
        }
        if (p.nsplit > 1 && half == 0 && head_ok) {
            p.part_ml[(prow_base + head) * 2] = m_run;
            p.part_ml[(prow_base + head) * 2 + 1] = l_run;
        }
    }
}

// Merges the key splits of one query row: out = sum_s w_s O_s / sum_s w_s with w_s = l_s 2^(m_s - m)
// and O_s the split's normalised fp16 partial (all zeros for an empty split, whose weight is zero).
// One thread per (row, head, 8 value channels); splits are taken eight at a time with all their loads
// in flight together.
__global__ __launch_bounds__(256) void sfa_combine_kernel(const SfaParams p)
{
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)p.T * p.NQ * (DN / 8);
    if (gid >= total) return;
    const int c8 = (int)(gid % (DN / 8));
    const size_t th = gid / (DN / 8);
    const int head = (int)(th % p.NQ);
    const int t = (int)(th / p.NQ);
    const size_t prow0 = (size_t)t * p.nsplit * p.NQ + head;       // split s: prow0 + s * NQ
    const f32x2 *ml = reinterpret_cast<const f32x2 *>(p.part_ml);

    float m = -INFINITY;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        f32x2 v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = ml[prow0 + (size_t)(s0 + e < p.nsplit ? s0 + e : p.nsplit - 1) * p.NQ];
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (v[e][1] > 0.f) m = fmaxf(m, v[e][0]);
    }
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        f32x2 v[8];
        f16x8 hv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const size_t prow = prow0 + (size_t)(s0 + e < p.nsplit ? s0 + e : p.nsplit - 1) * p.NQ;
            v[e] = ml[prow];
            hv[e] = *reinterpret_cast<const f16x8 *>(p.part_o + prow * DN + 8 * c8);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool live = s0 + e < p.nsplit && v[e][1] > 0.f;
            const float wgt = live ? v[e][1] * __builtin_amdgcn_exp2f(v[e][0] - m) : 0.f;
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[c] += wgt * (float)hv[e][c];
            wsum += wgt;
        }
    }
    const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
    u32x4 outv;
#pragma unroll
    for (int e = 0; e < 4; ++e) outv[e] = pack_bf16x2(acc[2 * e] * inv, acc[2 * e + 1] * inv);
    *reinterpret_cast<u32x4 *>(p.out + ((size_t)t * p.NQ + head) * DN + 8 * c8) = outv;
}

}  // namespace

hipError_t sfa_launch(const SfaParams &p, hipStream_t stream)
{
    const int rows8 = (p.T + 7) / 8 * 8;
    const unsigned grid = (unsigned)(rows8 * p.hgroups * p.nsplit);
    if (p.kn_bf16) {
        switch (p.waves) {
        case 1: hipLaunchKernelGGL((sfa_decode_kernel<1, false>), dim3(grid), dim3(64), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((sfa_decode_kernel<2, false>), dim3(grid), dim3(128), 0, stream, p); break;
        default: hipLaunchKernelGGL((sfa_decode_kernel<4, false>), dim3(grid), dim3(256), 0, stream, p); break;
        }
    } else {
        switch (p.waves) {
        case 1: hipLaunchKernelGGL((sfa_decode_kernel<1, true>), dim3(grid), dim3(64), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((sfa_decode_kernel<2, true>), dim3(grid), dim3(128), 0, stream, p); break;
        default: hipLaunchKernelGGL((sfa_decode_kernel<4, true>), dim3(grid), dim3(256), 0, stream, p); break;
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.nsplit > 1) {
        const size_t total = (size_t)p.T * p.NQ * (DN / 8);
        hipLaunchKernelGGL(sfa_combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace pto
