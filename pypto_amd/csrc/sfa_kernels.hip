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

template <int NW>
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
    // memory each such load touches 32 rows; instead the workgroup's heads are copied with coalesced
    // 16-byte loads (all issued before the first is consumed) into the LDS pool, 1168 bytes per head,
    // and every wave picks its fragments from there.  Heads past NQ read the last head and are never
    // stored.
    bf16x8 qf[KSTEPS];
    {
        constexpr int CHUNKS = D / 8;                         // 72 16-byte chunks per head
        constexpr int HEADS_WG = 32 * NW;
        constexpr int ITERS = (HEADS_WG * CHUNKS) / (NW * 64);   // 36
        u32x4 qtmp[ITERS];
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int c = tid + i * NW * 64;
            const int hl = c / CHUNKS;
            const int part = c - hl * CHUNKS;
            int hd = hg * HEADS_WG + hl;
            hd = hd < p.NQ ? hd : p.NQ - 1;
            const size_t qrow = (size_t)t * p.NQ + hd;
            const uint16_t *src = part < DN / 8 ? p.q_nope + qrow * DN + 8 * part : p.q_rope + qrow * DR + 8 * (part - DN / 8);
            qtmp[i] = *reinterpret_cast<const u32x4 *>(src);
        }
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int c = tid + i * NW * 64;
            const int hl = c / CHUNKS;
            *reinterpret_cast<u32x4 *>(pool + hl * PITCH + 8 * (c - hl * CHUNKS)) = qtmp[i];
        }
        __syncthreads();
        const uint16_t *qrow = pool + (w * 32 + col) * PITCH + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8 *>(qrow + 16 * ks);
        __syncthreads();                                      // the pool is free again
    }

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
    auto issue_loads = [&](const int kt) {
        const int *rtab = rows_lds + (kt - k_begin) + w * (KT / NW) + half * NP;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int row = rtab[i];
            raw[i] = *reinterpret_cast<const i32x4 *>(p.kn + (size_t)row * DN + 16 * col);
            rsc[i] = p.ksc[(size_t)row * 4 + (col >> 3)];
        }
#pragma unroll
        for (int i = 0; i < RP; ++i) {
            const int e = tid + i * NW * 64;
            const int row = rows_lds[(kt - k_begin) + (e >> 3)];
            rrope[i] = *reinterpret_cast<const u32x4 *>(p.kr + (size_t)row * DR + 8 * (e & 7));
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
            if (hidx < HALVES) {
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

    __syncthreads();                       // row table complete
    if (k_begin < k_end) {
        issue_loads(k_begin);
        store_tile(tile0);
    }
    __syncthreads();
    // All global loads issued so far (Q^T fragments, first tile) are complete from here on, so that
    // inside the loop the only outstanding vector-memory operations are the next tile's gather and
    // the compiler's wait counts do not serialise it with the matrix products.
    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0), expcnt and lgkmcnt unconstrained

    int it = 0;
    for (int kt = k_begin; kt < k_end; kt += KT, ++it) {
        const uint16_t *cur_tile = (it & 1) ? tile1 : tile0;
        uint16_t *nxt_tile = (it & 1) ? tile0 : tile1;
        issue_loads(kt + KT);                    // next tile (or the padding tile): in flight during the products

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

// ------------------------------------------------------------------ pipelined kernel, 128 heads
//
// Same decomposition and numerics as sfa_decode_kernel<4>, re-scheduled so that the matrix cores, the
// LDS and the vector ALU work at the same time.  Per tile n every wave runs two phases:
//   A  S(n+1) = K(n+1) . Q^T        (36 matrix products)  with the de-quantisation of tile n+2
//   B  O^T   += V(n)^T . P(n)^T     (32 matrix products)  with the softmax of S(n+1)
// with a barrier after each.  For the first product a wave owns 32 heads (Q^T fragments in registers,
// the whole K tile read from LDS); for the second it owns 128 value channels of ALL 128 heads, so it
// reads only its quarter of V^T and takes P^T -- 8 KiB per tile, exchanged through LDS -- as the
// other operand.  That halves the LDS traffic of the second product, which is what bounds the loop.  Tiles travel  cache --(LDS-DMA, four tiles ahead)--> int8 staging  --(phase A,
// two tiles ahead)--> bf16 tile --> phase A (K) and, one iteration later, phase B (V).  A wave
// stages and de-quantises the same eight keys of every tile, so the staging buffers need no barrier;
// the rope part of a row is bf16 already and is requested straight into the buffer phase A reads.
//
// LDS (bytes):  3 bf16 tiles of 32 x 520 (nope part; 1040 B pitch)      99840
//               4 rope buffers of 32 x 64 bf16 (16-byte chunk c of key k at position c ^ (k & 7))
//               2 int8 staging buffers of 32 x 512, 2 x 32 x 4 fp32 scales
//               P^T of the current tile, per-head rescale factors
//               row table of the split (logical position -> cache row), at most 1024 keys
// The prologue borrows the tile area to stage Q^T in two passes (nope dims 0..255, then 256..511 and
// the rope dims), every head row with its 16-byte chunks XOR-swizzled by the head number.
namespace pl {
constexpr int NPITCH = DN + 8;                                     // tile row pitch in elements
constexpr int TILE_BYTES = KT * NPITCH * 2;                        // 33280
constexpr int ROPE_BYTES = KT * DR * 2;                            // 4096
constexpr int STG_BYTES = KT * DN;                                 // 16384
constexpr int SC_BYTES = KT * 16;                                  // 512
constexpr int OFF_TILE = 0;
constexpr int OFF_ROPE = OFF_TILE + 3 * TILE_BYTES;
constexpr int OFF_STG = OFF_ROPE + 4 * ROPE_BYTES;
constexpr int OFF_SC = OFF_STG + 2 * STG_BYTES;
constexpr int P_BYTES = 2 * 2 * 128 * 16;                          // P^T of one tile: [16-key step][half][head] x 16 B
constexpr int OFF_P = OFF_SC + 2 * SC_BYTES;
constexpr int OFF_ALPHA = OFF_P + P_BYTES;                         // 128 rescale factors (later 1/l), 2 flags
constexpr int OFF_ROWS = OFF_ALPHA + 128 * 4 + 16;
constexpr int LDS_BYTES = OFF_ROWS + (SFA_PIPE_MAX_CHUNK + KT) * 4;
constexpr int QREGION = 20 * 1024;                                 // Q^T staging per wave: 16 KiB nope half + 4 KiB rope
static_assert(4 * QREGION <= 3 * TILE_BYTES, "Q staging must fit in the tile area");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
}  // namespace pl

typedef __attribute__((address_space(3))) uint8_t lds_byte_t;

// One LDS-DMA request: lane i's 16 bytes at gaddr land at lds_dst + 16*i.  lds_dst is wave-uniform.
// Written as assembly so that the compiler tracks none of these requests: the explicit vmcnt waits of
// the kernel decide how long they stay outstanding.
__device__ __forceinline__ void dma16(const void *gaddr, const uint32_t lds_dst)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gaddr), "s"(dst) : "memory", "m0");
}
// the same with a wave-uniform base address and a 32-bit byte offset per lane
__device__ __forceinline__ void dma16_base(const void *base, const uint32_t lane_off, const uint32_t lds_dst)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(dst) : "memory", "m0");
}
// the same for lanes 0..7 only (128 bytes)
__device__ __forceinline__ void dma16_low8(const void *gaddr, const uint32_t lds_dst)
{
    uint64_t saved;
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    asm volatile("s_mov_b64 %0, exec\n\t"
                 "s_mov_b64 exec, 0xff\n\t"
                 "s_mov_b32 m0, %2\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, off\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(gaddr), "s"(dst)
                 : "memory", "m0");
}

__global__ __launch_bounds__(256) void sfa_decode_pipelined_kernel(const SfaParams p)
{
    using namespace pl;
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];
    int *const rows_lds = reinterpret_cast<int *>(lds + OFF_ROWS);

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l = tid & 63;
    const int half = l >> 5;
    const int col = l & 31;
    const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lds_byte_t *)lds);

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
    const int n_valid = k_end > k_begin ? k_end - k_begin : 0;
    const int nt = (n_valid + KT - 1) / KT;                     // tiles of this split

    const int head = hg * 128 + w * 32 + col;
    const bool head_ok = head < p.NQ;

    // requests this wave's eight keys of tile m: rope (one request), scales (lanes 0..7), nope (four)
    auto request_tile = [&](const int m) {
        const int *rt = rows_lds + m * KT + 8 * w;
        {
            const int kk = l >> 3;
            dma16(p.kr + (size_t)rt[kk] * DR + 8 * ((l & 7) ^ kk), lds0 + OFF_ROPE + (m & 3) * ROPE_BYTES + w * 1024);
        }
        dma16_low8(p.ksc + (size_t)rt[l & 7] * 4, lds0 + OFF_SC + (m & 1) * SC_BYTES + w * 128);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dma16(p.kn + (size_t)rt[2 * i + half] * DN + 16 * col, lds0 + OFF_STG + (m & 1) * STG_BYTES + w * (8 * DN) + i * 1024);
    };
    // De-quantisation of key kk (0..7) of this wave's share of tile m into tile buffer tb, in two
    // halves: the staged bytes and the scale are read one step before they are converted, so that no
    // step waits for its own LDS reads.
    u32x2 dq_raw;
    float dq_sc;
    auto dequant_read = [&](const int m, const int kk) {
        const int key = 8 * w + kk;
        dq_raw = *reinterpret_cast<const u32x2 *>(lds + OFF_STG + (m & 1) * STG_BYTES + key * DN + 8 * l);
        dq_sc = *reinterpret_cast<const float *>(lds + OFF_SC + (m & 1) * SC_BYTES + key * 16 + 4 * (l >> 4));
    };
    // The same as a piece of vector work for the 36 slots of the S^T product (see gemm1): slot ks
    // converts quarter ks % 4 of key ks / 4; dequant_read(m, 0) must have been issued before.
    u32x2 dqm_raw;
    float dqm_sc, dqm_bias;
    u32x4 dqm_out;
    uint32_t dqm_v = 0;
    auto dequant_micro = [&](const int ks, const int m, const int tb) {
        const int g = ks >> 2, e = ks & 3;
        if (g >= 8) return;
        if (e == 0) {
            dqm_raw = dq_raw;
            dqm_sc = dq_sc;
            if (g + 1 < 8) dequant_read(m, g + 1);
            dqm_bias = -128.0f * dqm_sc;
        }
        if ((e & 1) == 0) dqm_v = dqm_raw[e >> 1] ^ 0x80808080u;
        // same arithmetic as dequant8: fma(float(byte + 128), sc, -128*sc) rounds x*sc once
        const float f0 = __builtin_fmaf((float)((dqm_v >> (16 * (e & 1))) & 0xffu), dqm_sc, dqm_bias);
        const float f1 = __builtin_fmaf((float)((dqm_v >> (16 * (e & 1) + 8)) & 0xffu), dqm_sc, dqm_bias);
        dqm_out[e] = pack_bf16x2(f0, f1);
        if (e == 3)
            *reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(lds + OFF_TILE + tb * TILE_BYTES) + (8 * w + g) * NPITCH + 8 * l) = dqm_out;
    };
    // a whole tile share at once (pipeline fill): all reads first, then the conversions
    auto dequant_tile = [&](const int m, const int tb) {
        u32x2 raw[8];
        float sc[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int key = 8 * w + kk;
            raw[kk] = *reinterpret_cast<const u32x2 *>(lds + OFF_STG + (m & 1) * STG_BYTES + key * DN + 8 * l);
            sc[kk] = *reinterpret_cast<const float *>(lds + OFF_SC + (m & 1) * SC_BYTES + key * 16 + 4 * (l >> 4));
        }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
            dequant8((int)raw[kk][0], (int)raw[kk][1], sc[kk],
                     reinterpret_cast<uint16_t *>(lds + OFF_TILE + tb * TILE_BYTES) + (8 * w + kk) * NPITCH + 8 * l);
    };

    // ---- prologue.  Everything that does not depend on anything else is requested at once: the first
    // half of Q^T, the top-k indices of the split and the sequence's block-table row.  Then, as the
    // data arrives: Q^T half 1 -> registers, Q^T half 2 requested, row table built (LDS lookups),
    // tiles 0 and 1 requested, Q^T half 2 -> registers.
    //
    // Q^T fragments: lane (head, half) holds q[head][16*ks + 8*half .. +8], staged per wave (its own 32
    // heads) in two passes: nope chunks 0..31 of every head, then nope chunks 32..63 plus the 8 rope
    // chunks.  A nope request covers two heads (lane = 32*(head & 1) + position), a rope request
    // eight (lane = 8*(head & 7) + position); position pos of head h holds chunk pos ^ (h & 7), which
    // makes the fragment reads conflict-free.  The cache address is a wave-uniform base plus a
    // per-lane offset.  Heads past NQ read the last head and are never stored.
    bf16x8 qf[KSTEPS];
    const uint32_t qdst = lds0 + OFF_TILE + w * QREGION;
    const int q_head0 = hg * 128 + w * 32;
    const bool q_all = q_head0 + 32 <= p.NQ;                          // wave-uniform: all 32 heads exist
    auto request_q = [&](const int pass) {
        const size_t qrow0 = (size_t)t * p.NQ + q_head0;
        if (q_all) {
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
        const uint8_t *qn = lds + OFF_TILE + w * QREGION + col * 512;
        const uint8_t *qr = lds + OFF_TILE + w * QREGION + 16 * 1024 + col * 128;
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) qf[16 * pass + ks] = *reinterpret_cast<const bf16x8 *>(qn + (((2 * ks + half) ^ (col & 7)) << 4));
        if (pass == 1) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qf[32 + ks] = *reinterpret_cast<const bf16x8 *>(qr + (((2 * ks + half) ^ (col & 7)) << 4));
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);                           // lgkmcnt(0): the region may be overwritten
    };
    request_q(0);

    // top-k indices of the split (at most four per thread) and the block-table row.  Keys past k_end in
    // the last tile repeat the split's first key (finite data, masked out of the softmax).
    constexpr int IDX_PER_THREAD = SFA_PIPE_MAX_CHUNK / 256;
    int idxr[IDX_PER_THREAD];
#pragma unroll
    for (int q = 0; q < IDX_PER_THREAD; ++q) {
        const int i = tid + 256 * q;
        idxr[q] = i < nt * KT ? p.topk_idx[(size_t)t * p.topk + k_begin + (i < n_valid ? i : 0)] : 0;
    }
    int *const bt_lds = reinterpret_cast<int *>(lds + OFF_P);        // the P^T area is idle until the loop
    const bool bt_cached = p.maxblk <= P_BYTES / 4;
    if (bt_cached)
        for (int i = tid; i < p.maxblk; i += 256) bt_lds[i] = p.bt[(size_t)b * p.maxblk + i];
    // (the compiler waits for these loads before it uses them; requests complete in order, so the first
    // half of Q^T has landed by then as well)
    __syncthreads();
#pragma unroll
    for (int q = 0; q < IDX_PER_THREAD; ++q) {
        const int i = tid + 256 * q;
        if (i < nt * KT) {
            const int idx = idxr[q];
            int blk = idx / p.bs;
            blk = blk < 0 ? 0 : (blk >= p.maxblk ? p.maxblk - 1 : blk);
            const int phys = bt_cached ? bt_lds[blk] : p.bt[(size_t)b * p.maxblk + blk];
            long long row = (long long)phys * p.bs + (idx - (idx / p.bs) * p.bs);
            row = row < 0 ? 0 : (row >= p.kv_rows ? p.kv_rows - 1 : row);
            rows_lds[i] = (int)row;
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                               // vmcnt(0): Q^T half 1 (and all else) landed
    collect_q(0);
    request_q(1);
    __syncthreads();                                                  // row table complete
    if (nt > 0) request_tile(0);
    if (nt > 1) request_tile(1);
    if (nt > 1) __builtin_amdgcn_s_waitcnt(0x0F7C);                   // vmcnt(12): Q^T half 2 landed, tiles may be in flight
    else if (nt > 0) __builtin_amdgcn_s_waitcnt(0x0F76);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    collect_q(1);
    __syncthreads();                                                  // the tile area is free

    f32x16 o[DVB];
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    valu_to_mfma_fence();
    float m_run = -INFINITY;   // reference max, log2 domain
    float l_run = 0.f;         // running sum of exp2(s - m_run)

    // Issue order.  A wave issues in order and a matrix product occupies the matrix pipe for 32 cycles,
    // so the next product in program order stalls everything behind it: vector and LDS instructions
    // overlap with the matrix pipe only when they sit BETWEEN two products, about seven of them at
    // most.  Both phases are therefore written as "slots" -- one product, the operand reads of a later
    // product, one small piece of vector work -- and a scheduling barrier after every slot keeps the
    // compiler from regrouping them.

    // S^T of tile buffer tb / rope buffer rb: 36 slots; micro(ks) is the caller's piece of vector work.
    // Operand reads stay four products ahead.
    auto gemm1 = [&](const int tb, const int rb, f32x16 &s, auto &&micro) {
        const uint16_t *arow = reinterpret_cast<const uint16_t *>(lds + OFF_TILE + tb * TILE_BYTES) + col * NPITCH + 8 * half;
        const uint8_t *rrow = lds + OFF_ROPE + rb * ROPE_BYTES + col * (DR * 2);
        bf16x8 fa[2][4];
        auto read_a = [&](const int ks) -> bf16x8 {
            return ks < DN / 16 ? *reinterpret_cast<const bf16x8 *>(arow + 16 * ks)
                                : *reinterpret_cast<const bf16x8 *>(rrow + (((2 * (ks - DN / 16) + half) ^ (col & 7)) << 4));
        };
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) fa[0][e] = read_a(e);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[(ks >> 2) & 1][ks & 3], qf[ks], s, 0, 0, 0);
            if (ks + 4 < KSTEPS) fa[((ks >> 2) + 1) & 1][ks & 3] = read_a(ks + 4);
            micro(ks);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Online softmax of the S^T block in s (already masked and still unscaled), cut into 32 slots that
    // ride between the matrix products of the PV phase.  Lane (head, half) holds keys
    // kt + 8*(r/4) + 4*half + r%4.  The reference max follows the true max lazily: probabilities may
    // reach 2^RESCALE_TAU, which fp32 sums and bf16 P hold without loss, and the accumulators are
    // rescaled (by the caller, before the tile's PV products) only on a jump.  A tile entirely past
    // k_end leaves the running state as it is: every probability is exp2(-inf) = 0.
    float sm_mx = 0.f, sm_mnew = 0.f, sm_alpha = 1.0f, sm_lsum = 0.f;
    bool sm_rescale = false;
    auto softmax_micro = [&](const int m, f32x16 &s, bf16x8 (&pf)[2]) {
        if (m < 4) {                                            // scale
#pragma unroll
            for (int r = 4 * m; r < 4 * m + 4; ++r) s[r] *= p.scale_log2;
        } else if (m < 8) {                                     // running max
            const int r = 4 * (m - 4);
            const float part = fmaxf(fmaxf(s[r], s[r + 1]), fmaxf(s[r + 2], s[r + 3]));
            sm_mx = m == 4 ? part : fmaxf(sm_mx, part);
        } else if (m == 8) {                                    // both half-waves, then the lazy reference
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(sm_mx), __float_as_uint(sm_mx), false, false);
            sm_mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
            const bool upd = sm_mx > m_run + RESCALE_TAU;       // always true on the first tile (m_run = -inf)
            sm_mnew = upd ? sm_mx : m_run;
            sm_rescale = upd && l_run > 0.f;                    // nothing accumulated yet: nothing to rescale
        } else if (m == 9) {
            sm_alpha = sm_mnew > m_run ? __builtin_amdgcn_exp2f(m_run - sm_mnew) : 1.0f;
        } else if (m < 26) {                                    // one exponential per slot
            const int r = m - 10;
            s[r] = __builtin_amdgcn_exp2f(s[r] - sm_mnew);
        } else if (m < 28) {                                    // row sum
            const int r = 8 * (m - 26);
            const float part = ((s[r] + s[r + 1]) + (s[r + 2] + s[r + 3])) + ((s[r + 4] + s[r + 5]) + (s[r + 6] + s[r + 7]));
            sm_lsum = m == 26 ? part : sm_lsum + part;
        } else if (m == 28) {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(sm_lsum), __float_as_uint(sm_lsum), false, false);
            sm_lsum = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            l_run = l_run * sm_alpha + sm_lsum;
            m_run = sm_mnew;
        } else if (m < 31) {                                    // P^T fragments
            const int kk = m - 29;
            u32x4 pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = pack_bf16x2(s[8 * kk + 2 * e], s[8 * kk + 2 * e + 1]);
            pf[kk] = __builtin_bit_cast(bf16x8, pk);
        }
    };
    // keys past k_end of the tile starting at kt
    auto mask_tail = [&](const int kt, f32x16 &s) {
        if (kt + KT > k_end) {                   // only the split's last tile (or a tile past it)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (kt + 8 * (r >> 2) + 4 * half + (r & 3) >= k_end) s[r] = -INFINITY;
        }
    };

    // ---- pipeline fill: tile 0 de-quantised, S(0) with the de-quantisation of tile 1 between its
    // products, tiles 2 and 3 requested as soon as their staging buffers are free, softmax of S(0)
    f32x16 s;
    bf16x8 pf_cur[2], pf_next[2];
    if (nt > 0) {
        if (nt > 1) __builtin_amdgcn_s_waitcnt(0x0F76);               // vmcnt(6): tile 0 staged, tile 1 may be in flight
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        dequant_tile(0, 0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);
        if (nt > 2) request_tile(2);
        __syncthreads();
        if (nt > 2) __builtin_amdgcn_s_waitcnt(0x0F76);               // tile 1 staged
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        dequant_read(1, 0);
        gemm1(0, 0, s, [&](const int ks) { dequant_micro(ks, 1, 1); });
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);
        if (nt > 3) request_tile(3);
        mask_tail(k_begin, s);
#pragma unroll
        for (int m = 0; m < 32; ++m) softmax_micro(m, s, pf_cur);
        sm_rescale = false;
        __syncthreads();                                              // tile 1 complete
    }

    float *const alpha_tab = reinterpret_cast<float *>(lds + OFF_ALPHA);
    int *const resc_flag = reinterpret_cast<int *>(lds + OFF_ALPHA + 128 * 4);
    if (tid < 2) resc_flag[tid] = 0;

    int tb_cur = 0;                          // tile buffer of tile n: n % 3
    for (int n = 0; n < nt; ++n) {
        const int tb_next = tb_cur == 2 ? 0 : tb_cur + 1;
        const int tb_fill = tb_next == 2 ? 0 : tb_next + 1;

        // P(n)^T and the rescale factors found by the softmax of S(n) go to LDS for all waves
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
            *reinterpret_cast<bf16x8 *>(lds + OFF_P + (((kk * 2 + half) * 128 + 32 * w + col) << 4)) = pf_cur[kk];
        if (half == 0) alpha_tab[32 * w + col] = sm_alpha;
        if (__any(sm_rescale) && l == 0) resc_flag[n & 1] = 1;
        if (tid == 0) resc_flag[(n + 1) & 1] = 0;

        // ---- phase A: S(n+1) with the de-quantisation of this wave's keys of tile n+2 (one key per
        // four products), then the request for tile n+4 into the staging buffer just read.
        // Past the last tile the products run on stale data; the softmax below masks all of it.
        if (n + 3 < nt) __builtin_amdgcn_s_waitcnt(0x0F76);      // vmcnt(6): tile n+2 staged, n+3 may be in flight
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        dequant_read(n + 2, 0);
        gemm1(tb_next, (n + 1) & 3, s, [&](const int ks) { dequant_micro(ks, n + 2, tb_fill); });
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);                      // lgkmcnt(0): the staging buffer has been read
        if (n + 4 < nt) request_tile(n + 4);
        __syncthreads();

        // ---- phase B: O^T[128 channels of this wave][128 heads] += V(n)^T . P(n)^T with the softmax of
        // S(n+1).  Product m = 16*kk + 4*i + hb: 16-key step kk, channel block i, head block hb.
        if (__builtin_amdgcn_readfirstlane(resc_flag[n & 1]) != 0) {   // some head's reference max jumped
            float al[4];
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) al[hb] = alpha_tab[32 * hb + col];
            mfma_to_valu_fence();
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int hb = 0; hb < 4; ++hb) acc_scale(o[4 * i + hb], al[hb]);
            valu_to_mfma_fence();
        }
        {
            const int kt_next = k_begin + (n + 1) * KT;
            const uint16_t *vbase = reinterpret_cast<const uint16_t *>(lds + OFF_TILE + tb_cur * TILE_BYTES) +
                                    (4 * half + ((l & 15) >> 2)) * NPITCH + 16 * ((l >> 4) & 1) + 4 * (l & 3) + 128 * w;
            const uint8_t *pbase = lds + OFF_P + ((half * 128 + col) << 4);
            bf16x8 bq[2][4];
            s16x4 av[2][2];
            auto read_v = [&](const int m, s16x4 (&v)[2]) {     // V^T operand of products m .. m+3
                const uint16_t *a0 = vbase + (16 * (m >> 4)) * NPITCH + 32 * ((m >> 2) & 3);
                v[0] = lds_read_tr16(a0);
                v[1] = lds_read_tr16(a0 + 8 * NPITCH);
            };
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) bq[0][hb] = *reinterpret_cast<const bf16x8 *>(pbase + ((32 * hb) << 4));
            read_v(0, av[0]);
            mask_tail(kt_next, s);
#pragma unroll
            for (int m = 0; m < 32; ++m) {
                const int kk = m >> 4, i = (m >> 2) & 3, hb = m & 3;
                const s16x8 a = __builtin_shufflevector(av[(m >> 2) & 1][0], av[(m >> 2) & 1][1], 0, 1, 2, 3, 4, 5, 6, 7);
                acc_mfma(o[4 * i + hb], __builtin_bit_cast(bf16x8, a), bq[kk][hb]);
                if (hb == 0 && m + 4 < 32) read_v(m + 4, av[((m >> 2) + 1) & 1]);
                if (m < 4) bq[1][m] = *reinterpret_cast<const bf16x8 *>(pbase + ((2 * 128 + 32 * m) << 4));
                softmax_micro(m, s, pf_next);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
        pf_cur[0] = pf_next[0];
        pf_cur[1] = pf_next[1];
        tb_cur = tb_next;
    }

    // ---- epilogue.  Wave w holds value channels 128*w .. +127 of all 128 heads: accumulator
    // o[4*i + hb], lane (head, half) = channels 128*w + 32*i + 8*(r/4) + 4*half + r%4 of head 32*hb + head.
    // One head block at a time, scaled by 1/l and rounded to the 16-bit output type, goes through the
    // wave's slice of the (now idle) tile area, so that 32 lanes write 256 contiguous bytes of one
    // head.  The 1/l factors of all heads are shared through LDS.
    mfma_to_valu_fence();
    {
        float *stage = reinterpret_cast<float *>(lds) + w * (32 * 128);
        float *inv_tab = alpha_tab;
        const size_t prow_base = ((size_t)t * p.nsplit + sp) * p.NQ;
        if (half == 0) inv_tab[32 * w + col] = l_run > 0.f ? 1.0f / l_run : 0.f;
        __syncthreads();
        // FINAL: bf16 result rows; otherwise fp16 partial of a key split (O / l of the split, merged by
        // the combine kernel with weights l * 2^(m - m_max); O / l is a convex combination of
        // de-quantised V rows, so it stays finite in fp16 as long as |int8 * scale| < 65504).
        // ALL: every head of the block exists, so the stores need no predicate.  Both are uniform and
        // resolved outside the loops: scalar branches inside them cost more than the work.
        auto drain = [&](auto hb_tag, auto final_tag, auto all_tag) {
            constexpr int HB = decltype(hb_tag)::value;
            constexpr bool FINAL = decltype(final_tag)::value;
            constexpr bool ALL = decltype(all_tag)::value;
            const int head_base = hg * 128 + 32 * HB;
            uint16_t *dst0 = FINAL ? p.out + ((size_t)t * p.NQ + head_base + half) * DN + 128 * w + 4 * col
                                   : p.part_o + (prow_base + head_base + half) * DN + 128 * w + 4 * col;
            const float inv = inv_tab[32 * HB + col];               // this lane's head of the block
            // staged as 16-bit values: 8-byte chunk c (4 channels) of head h at chunk c ^ (h & 15)
            uint8_t *st = reinterpret_cast<uint8_t *>(stage);
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const f32x16 &acc = o[4 * b4 + HB];
                    const float v0 = acc[4 * q4] * inv, v1 = acc[4 * q4 + 1] * inv, v2 = acc[4 * q4 + 2] * inv, v3 = acc[4 * q4 + 3] * inv;
                    u32x2 pk;
                    pk[0] = FINAL ? pack_bf16x2(v0, v1) : pack_f16x2(v0, v1);
                    pk[1] = FINAL ? pack_bf16x2(v2, v3) : pack_f16x2(v2, v3);
                    *reinterpret_cast<u32x2 *>(st + col * 256 + (((8 * b4 + 2 * q4 + half) ^ (col & 15)) << 3)) = pk;
                }
#pragma unroll 1
            for (int pq = 0; pq < 2; ++pq) {
                u32x2 rv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int hl = 2 * (8 * pq + e) + half;
                    rv[e] = *reinterpret_cast<const u32x2 *>(st + hl * 256 + ((col ^ (hl & 15)) << 3));
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int hl = 2 * (8 * pq + e) + half;
                    if (ALL || head_base + hl < p.NQ)
                        *reinterpret_cast<u32x2 *>(dst0 + (size_t)(hl - half) * DN) = rv[e];
                }
            }
        };
        auto drain_block = [&](auto hb_tag) {
            const bool all_heads = hg * 128 + 32 * decltype(hb_tag)::value + 32 <= p.NQ;
            if (p.nsplit == 1) {
                if (all_heads) drain(hb_tag, std::true_type{}, std::true_type{});
                else drain(hb_tag, std::true_type{}, std::false_type{});
            } else {
                if (all_heads) drain(hb_tag, std::false_type{}, std::true_type{});
                else drain(hb_tag, std::false_type{}, std::false_type{});
            }
        };
        drain_block(std::integral_constant<int, 0>{});
        drain_block(std::integral_constant<int, 1>{});
        drain_block(std::integral_constant<int, 2>{});
        drain_block(std::integral_constant<int, 3>{});
        if (p.nsplit > 1 && half == 0 && head_ok) {
            p.part_ml[(prow_base + head) * 2] = m_run;
            p.part_ml[(prow_base + head) * 2 + 1] = l_run;
        }
    }
}

// Merges the key splits of one query row: out = sum_s w_s O_s / sum_s w_s with w_s = l_s 2^(m_s - m)
// and O_s the split's normalised fp16 partial.  One thread per (row, head, 8 value channels).
__global__ __launch_bounds__(256) void sfa_combine_kernel(const SfaParams p)
{
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)p.T * p.NQ * (DN / 8);
    if (gid >= total) return;
    const int c8 = (int)(gid % (DN / 8));
    const size_t th = gid / (DN / 8);
    const int head = (int)(th % p.NQ);
    const int t = (int)(th / p.NQ);
    float m = -INFINITY;
    for (int s = 0; s < p.nsplit; ++s) {
        const size_t prow = ((size_t)t * p.nsplit + s) * p.NQ + head;
        if (p.part_ml[prow * 2 + 1] > 0.f) m = fmaxf(m, p.part_ml[prow * 2]);
    }
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
    for (int s = 0; s < p.nsplit; ++s) {
        const size_t prow = ((size_t)t * p.nsplit + s) * p.NQ + head;
        const float ls = p.part_ml[prow * 2 + 1];
        if (ls > 0.f) {
            const float wgt = ls * __builtin_amdgcn_exp2f(p.part_ml[prow * 2] - m);
            const f16x8 hv = *reinterpret_cast<const f16x8 *>(p.part_o + prow * DN + 8 * c8);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += wgt * (float)hv[e];
            wsum += wgt;
        }
    }
    const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
    u32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = pack_bf16x2(acc[2 * e] * inv, acc[2 * e + 1] * inv);
    *reinterpret_cast<u32x4 *>(p.out + ((size_t)t * p.NQ + head) * DN + 8 * c8) = v;
}

}  // namespace

hipError_t sfa_launch(const SfaParams &p, hipStream_t stream)
{
    const int rows8 = (p.T + 7) / 8 * 8;
    const unsigned grid = (unsigned)(rows8 * p.hgroups * p.nsplit);
    switch (p.waves) {
    case 1: hipLaunchKernelGGL(sfa_decode_kernel<1>, dim3(grid), dim3(64), 0, stream, p); break;
    case 2: hipLaunchKernelGGL(sfa_decode_kernel<2>, dim3(grid), dim3(128), 0, stream, p); break;
    default: hipLaunchKernelGGL(sfa_decode_pipelined_kernel, dim3(grid), dim3(256), 0, stream, p); break;
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
