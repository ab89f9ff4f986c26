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

// Row i of a tile's score operand (and of the score accumulator) is key tile_row_of(i) of the tile: the two
// middle bits of i move below its two lowest.  A transposing V^T read then addresses keys r, r+4, r+8, r+12
// with each of its half-waves, four rows whose 64-byte pieces lie 16 banks apart at this pitch, instead of
// four neighbouring rows whose pieces overlap pairwise; any 16 consecutive keys, in whatever order, still
// serve the 16-byte score operand reads without a conflict.
__device__ __forceinline__ constexpr int tile_row_of(const int i)
{
    return (i & 16) | ((i & 3) << 2) | ((i >> 2) & 3);
}

// Four int8 (one dword) times one scale -> four bf16 in two registers.
// x*sc is formed as fma(float(x + 128), sc, -128*sc): the byte is biased to unsigned so that a single
// v_cvt_f32_ubyteN converts it, and the fused multiply-add rounds the exact product (x*sc) once, which
// is bit-identical to the rounded multiply (128*sc is exact).
__device__ __forceinline__ u32x2 dequant4(const uint32_t r, const float sc, const float bias /* -128 * sc */)
{
    const uint32_t v = r ^ 0x80808080u;
    const float f0 = __builtin_fmaf((float)(v & 0xffu), sc, bias);
    const float f1 = __builtin_fmaf((float)((v >> 8) & 0xffu), sc, bias);
    const float f2 = __builtin_fmaf((float)((v >> 16) & 0xffu), sc, bias);
    const float f3 = __builtin_fmaf((float)(v >> 24), sc, bias);
    u32x2 out;
    out[0] = pack_bf16x2(f0, f1);
    out[1] = pack_bf16x2(f2, f3);
    return out;
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

// First product into an O^T block: starts from zero, so the 256 accumulation registers need no clearing
// (256 writes in front of the key loop otherwise).
__device__ __forceinline__ void acc_mfma_first(f32x16 &acc, const bf16x8 a, const bf16x8 b)
{
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}

// S^T accumulator: kept in architectural registers by construction.  Left to the compiler it shares the
// first sixteen accumulation registers with the first O^T block, which is then copied out and back
// around every tile.  First product of a chain starts from zero; the chain is dependent products on one
// destination (no wait states needed between them); s_chain_done pads the matrix-write -> vector-read slot.
__device__ __forceinline__ void s_mfma_first(f32x16 &s, const bf16x8 a, const bf16x8 b)
{
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b));
}
__device__ __forceinline__ void s_mfma(f32x16 &s, const bf16x8 a, const bf16x8 b)
{
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b));
}
__device__ __forceinline__ void s_chain_done(f32x16 &s) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(s)); }

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

// both half-waves' values of x, in every lane: one register-to-register exchange (no LDS round trip)
__device__ __forceinline__ void both_halves(const float x, float &lo, float &hi)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

constexpr float RESCALE_TAU = 8.0f;   // log2 units: the reference max moves only when exceeded by 2^8

// QUANT: the latent part of a cache row is int8 with four fp32 scales and is de-quantised on the way into
// LDS; otherwise it is bf16 already (1024 bytes) and travels cache -> LDS tile directly by LDS-DMA.
template <int NW, bool QUANT>
__global__ __launch_bounds__(NW * 64) void sfa_decode_kernel(const SfaParams p)
{
    // One LDS pool.  Prologue: per-wave query staging regions (QREGION bytes each).  Loop: tile
    // buffers of KT rows -- while tile n is consumed from one, tile n+1 is de-quantised into the other
    // (int8 cache: out of a staging ring of raw rows above the tile buffers, filled by LDS-DMA two tiles
    // ahead); one barrier per tile.  Epilogue: per-wave transposition slices.
    constexpr int QREGION = 20 * 1024;                                 // per wave: 16 KiB nope half + 4 KiB rope
    constexpr int EPI_BYTES = 32 * 128 * 4;                            // per wave: 32 heads x 128 channels fp32
    constexpr int TILES_BYTES = 2 * KT * PITCH * 2;
    constexpr int WAVE_BYTES = NW * (QREGION > EPI_BYTES ? QREGION : EPI_BYTES);
    constexpr int STG_NOPE = KT * DN;                                  // bytes of one staged tile: int8 rows,
    constexpr int STG_SCALE = KT * 16;                                 // four fp32 scales per row,
    constexpr int STG_ROPE = KT * DR * 2;                              // bf16 rope rows
    constexpr int STG_BYTES = STG_NOPE + STG_SCALE + STG_ROPE;
    constexpr int STG_SLOTS = 2;
    constexpr int STG_BASE = TILES_BYTES > WAVE_BYTES ? TILES_BYTES : WAVE_BYTES;   // above everything else in the pool
    constexpr int POOL_BYTES = STG_BASE + (QUANT ? STG_SLOTS * STG_BYTES : 0);
    static_assert(STG_BASE % 16 == 0 && STG_BYTES % 16 == 0, "LDS-DMA destinations are 16-byte aligned");
    __shared__ __attribute__((aligned(16))) uint16_t pool[POOL_BYTES / 2];
    __shared__ int rows_lds[SFA_MAX_CHUNK + 3 * KT];
    uint16_t *const tile0 = pool;
    uint16_t *const tile1 = pool + KT * PITCH;

    const int tid = threadIdx.x;
    const int w = tid >> 6;
    const int l = tid & 63;
    const int half = l >> 5;
    const int col = l & 31;

    // Workgroups of one query row share an XCD (consecutive workgroup ids rotate over the 8 XCDs): row t is row
    // slot t / 8 of XCD t % 8.  The first whole_slots row slots of every XCD are rows taken by one workgroup each
    // (per head group), the others are split over nsplit workgroups: a launch of more rows than compute units
    // runs its full rounds of whole rows first and deals the rows left over out in pieces.
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int wslots = p.whole_slots * p.hgroups;
    int rslot, within, nsplit;
    if (slot < wslots) {
        rslot = slot / p.hgroups;
        within = slot - rslot * p.hgroups;
        nsplit = 1;
    } else {
        const int per_row = p.hgroups * p.nsplit;
        rslot = p.whole_slots + (slot - wslots) / per_row;
        within = (slot - wslots) % per_row;
        nsplit = p.nsplit;
    }
    const int t = rslot * 8 + xcd;
    if (t >= p.T) return;
    const int hg = within / nsplit;
    const int sp = within % nsplit;
    const int b = t / p.S1;
    const int s1i = t - b * p.S1;

    // The sequence length is asked for here and looked at only after the first requests below are on their
    // way: the memory latency of this load would otherwise stand in front of everything else.
    const int act_b = p.act[b];
    // keys [kb, ke) of a row with n selected keys that this split takes
    auto split_keys = [&](const int n, int &kb, int &ke) {
        const int ntile = (n + KT - 1) / KT;
        const int tiles_per_split = (ntile + nsplit - 1) / nsplit;
        kb = sp * tiles_per_split * KT;
        ke = kb + tiles_per_split * KT;
        ke = ke > n ? n : ke;
    };

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
    // pending: the number of younger requests of this wave that may still be in flight
    auto collect_q = [&](const int pass, auto pending) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(decltype(pending)::value));   // the pass has landed
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
    // logical position -> physical cache row for this split's keys.  The table is padded to an even
    // number of tiles plus two with the row of the split's first key: keys past k_end are then loaded
    // like any other (finite data) and masked out of the softmax, and the loop can prefetch two tiles
    // ahead unconditionally -- no per-key and no per-tile branches.
    //
    // The translation is a chain of two dependent loads (selected position, then its page in the block
    // table) ahead of the gather itself.  When the table fits two entries per thread both loads travel
    // as LDS-DMA requests between the Q^T passes, waited for by count, so that the chain runs beside
    // the Q^T staging instead of after it; each lane handles the entries it requested itself.
    constexpr int FAST_ENTRIES = 2 * NW * 64;
    static_assert(2 * FAST_ENTRIES <= SFA_MAX_CHUNK + 3 * KT, "positions and pages of the short table share its memory");
    auto padded = [](const int n) { return n > 0 ? (n + 2 * KT - 1) / (2 * KT) * (2 * KT) + 2 * KT : 0; };
    const int wave_first = __builtin_amdgcn_readfirstlane(w) * 64;
    auto row_of = [&](const int idx, const int page) {
        long long row = (long long)page * p.bs + (idx - (idx / p.bs) * p.bs);
        row = row < 0 ? 0 : (row >= p.kv_rows ? p.kv_rows - 1 : row);
        return (int)row;
    };
    auto block_of = [&](const int idx) {
        const int blk = idx / p.bs;
        return blk < 0 ? 0 : (blk >= p.maxblk ? p.maxblk - 1 : blk);
    };
    auto request_positions = [&](const int kb, const int nv) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int i = tid + j * NW * 64;
            dma4(p.topk_idx + (size_t)t * p.topk + kb + (i < nv ? i : 0),
                 (uint32_t)(uintptr_t)(lds_byte_t *)(rows_lds + j * NW * 64 + wave_first));
        }
    };
    // A decoding row nearly always sees all topk selected keys.  The positions of this split are requested on
    // that assumption before the sequence length has arrived, which takes one memory latency out of the chain
    // length -> positions -> pages -> rows -> first tile; if the length says otherwise they are requested
    // again (same destinations; requests complete in order, so the later ones stand).
    int kb_s, ke_s;
    split_keys(p.topk, kb_s, ke_s);
    const int nv_s = ke_s - kb_s;
    const bool fast_s = nv_s > 0 && padded(nv_s) <= FAST_ENTRIES;              // uniform
    if (fast_s) request_positions(kb_s, nv_s);
    request_q(0);                                                             // 16 requests
    int cur = act_b - p.S1 + 1 + s1i;
    cur = cur < 0 ? 0 : (cur > p.topk ? p.topk : cur);
    int k_begin, k_end;
    split_keys(cur, k_begin, k_end);
    const int n_valid = k_end - k_begin;
    const int n_pad = padded(n_valid);
    const bool fast = n_valid > 0 && n_pad <= FAST_ENTRIES;                    // uniform
    const bool as_assumed = fast_s && k_begin == kb_s && n_valid == nv_s;     // uniform
    if (fast) {
        if (as_assumed) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(16));                        // the positions have landed
        } else {
            request_positions(k_begin, n_valid);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int i = tid + j * NW * 64;
            dma4(p.bt + (size_t)b * p.maxblk + block_of(rows_lds[i]),
                 (uint32_t)(uintptr_t)(lds_byte_t *)(rows_lds + FAST_ENTRIES + j * NW * 64 + wave_first));
        }
        collect_q(0, std::integral_constant<int, 2>{});
    } else {
        collect_q(0, std::integral_constant<int, 0>{});
    }
    request_q(1);                                                             // 20 requests
    if (fast) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(20));                            // the pages have landed
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int i = tid + j * NW * 64;
            rows_lds[i] = row_of(rows_lds[i], rows_lds[FAST_ENTRIES + i]);
        }
    } else {
        for (int i = tid; i < n_pad; i += NW * 64) {
            const int idx = p.topk_idx[(size_t)t * p.topk + k_begin + (i < n_valid ? i : 0)];
            rows_lds[i] = row_of(idx, p.bt[(size_t)b * p.maxblk + block_of(idx)]);
        }
    }

    // the first tile's products start the accumulators from zero (acc_mfma_first); they are cleared beforehand
    // only when there is no first tile
    f32x16 o[DVB];
    if (k_begin >= k_end) {
#pragma unroll
        for (int i = 0; i < DVB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
        valu_to_mfma_fence();
    }
    float m_run = -INFINITY;   // reference max, log2 domain
    float l_run = 0.f;         // running sum of exp2(s - m_run)

    // Gather.  Wave w owns keys w*KT/NW .. +KT/NW of every tile.
    //   QUANT: the rows travel cache -> LDS staging area by LDS-DMA two tiles ahead of their use (no
    //   registers are held across the products): per tile and wave KPW/2 requests of two int8 rows
    //   (512 B each), one of the KPW scale quadruples, KPW/8 of eight rope rows (128 B each).  The
    //   staging ring of two tiles sits above the tile buffers; a wave
    //   de-quantises exactly what it requested, so its own wait count is all the ordering needed.
    //   bf16 cache: rows go straight into the tile buffer (one request per key), one tile ahead.
    constexpr int NP = KT / (2 * NW);
    constexpr int RP = (KT * (DR / 8)) / (NW * 64);
    constexpr int KPW = KT / NW;                                  // keys per wave and tile
    constexpr int DMA_PER_TILE = KPW / 2 + 1 + (KPW + 7) / 8;     // requests per wave and tile
    static_assert(2 * DMA_PER_TILE <= 48, "two tiles of requests stay outstanding");
    u32x4 rrope[RP];

    // Per-lane byte offsets into the pool, kept opaque to the optimiser: every LDS access of the
    // staged path is then "one of these registers + an immediate" instead of an address register of
    // its own (dozens of them, at the price of spilled Q^T fragments).
    const int wu = __builtin_amdgcn_readfirstlane(w);
    uint32_t fetch_off = STG_BASE + w * KPW * DN + 8 * l;                          // this lane's 8 staged bytes of a key
    uint32_t scale_off = STG_BASE + STG_NOPE + w * KPW * 16 + 4 * (l >> 4);          // their scale
    uint32_t ropes_off = STG_BASE + STG_NOPE + STG_SCALE + 16 * (w * KPW * 8 + l);   // staged rope piece
    uint32_t emit_off = (w * KPW * PITCH) * 2 + 16 * l;                              // the 8 de-quantised channels
    uint32_t ropee_off = ((w * KPW + (l >> 3)) * PITCH + DN + 8 * (l & 7)) * 2;      // rope piece in the tile
    if (QUANT) asm volatile("" : "+v"(fetch_off), "+v"(scale_off), "+v"(ropes_off), "+v"(emit_off), "+v"(ropee_off));
    uint8_t *const pool_b = reinterpret_cast<uint8_t *>(pool);

    // Request k of a tile (QUANT only): k < KPW/2 two int8 rows, k == KPW/2 the scale quadruples, then
    // eight rope rows each.  stage_row reads the cache row number a lane needs for request k,
    // stage_request issues it.
    auto stage_row = [&](const int kt, const int k) {
        const int *rtab = rows_lds + (kt - k_begin) + wu * KPW;
        if (k < KPW / 2) return rtab[2 * k + half];
        if (k == KPW / 2) return rtab[l & (KPW - 1)];
        return rtab[8 * (k - KPW / 2 - 1) + (l >> 3)];
    };
    auto stage_request = [&](const int slot, const int k, const int row) {
        const uint32_t dst = (uint32_t)(uintptr_t)(lds_byte_t *)pool_b + STG_BASE + slot * STG_BYTES;
        if (k < KPW / 2) {
            dma16(p.kn + (size_t)row * p.kn_pitch + 16 * col, dst + (wu * KPW + 2 * k) * DN);
        } else if (k == KPW / 2) {
            dma16_lanes(p.ksc + (size_t)row * p.ksc_pitch, dst + STG_NOPE + wu * KPW * 16, (1ull << KPW) - 1ull);
        } else {
            dma16(p.kr + (size_t)row * p.kr_pitch + 16 * (l & 7),
                  dst + STG_NOPE + STG_SCALE + (wu * KPW + 8 * (k - KPW / 2 - 1)) * (DR * 2));
        }
    };
    auto stage_tile = [&](const int kt, const int slot) {          // a whole tile at once: the prologue
        int rows[DMA_PER_TILE];
#pragma unroll
        for (int k = 0; k < DMA_PER_TILE; ++k) rows[k] = stage_row(kt, k);
#pragma unroll
        for (int k = 0; k < DMA_PER_TILE; ++k) stage_request(slot, k, rows[k]);
    };
    auto issue_loads = [&](const int kt, uint16_t *buf) {          // bf16 cache only
        // one request per key: the 64 lanes' 16-byte pieces are the 1024 bytes of the row, in order
        const int *rtab = rows_lds + (kt - k_begin) + w * (KT / NW);
#pragma unroll
        for (int i = 0; i < KT / NW; ++i)
            dma16(p.kn + (size_t)rtab[i] * p.kn_pitch + 16 * l,
                  (uint32_t)(uintptr_t)(lds_byte_t *)(buf + (w * (KT / NW) + i) * PITCH));
#pragma unroll
        for (int i = 0; i < RP; ++i) {
            const int e = tid + i * NW * 64;
            const int row = rows_lds[(kt - k_begin) + (e >> 3)];
            rrope[i] = *reinterpret_cast<const u32x4 *>(p.kr + (size_t)row * p.kr_pitch + 16 * (e & 7));
        }
    };
    // De-quantisation of a staged tile, one eighth ("piece") at a time: fetch_piece reads the staged bytes
    // (eight per key and lane) and the key's scale into a few registers; emit_step (below) converts a quarter
    // of one half of them -- the lower four bytes are half 0, the upper four half 1, which also stores the
    // eight channels: the wave's 64 lanes write the 1024 contiguous bytes of the key's row in the tile
    // buffer (tile = 0 or 1).  Each piece is fetched a few products before its first half is converted.
    constexpr int PER = (KPW + 7) / 8;             // keys of this wave per piece
    u32x2 praw[2][QUANT ? PER : 1], plow[QUANT ? PER : 1];
    float pbias[QUANT ? PER : 1];
    float psc[2][QUANT ? PER : 1];
    auto fetch_piece = [&](const int piece, const int slot) {
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int i = piece * PER + q;         // key of this wave: a wave instruction covers its 512 bytes
            if (i < KPW) {
                praw[piece & 1][q] = *reinterpret_cast<const u32x2 *>(pool_b + fetch_off + (slot * STG_BYTES + i * DN));
                psc[piece & 1][q] = *reinterpret_cast<const float *>(pool_b + scale_off + (slot * STG_BYTES + i * 16));
            }
        }
    };
    auto fetch_rope = [&](const int slot) {
#pragma unroll
        for (int i = 0; i < RP; ++i)
            rrope[i] = *reinterpret_cast<const u32x4 *>(pool_b + ropes_off + (slot * STG_BYTES + i * 1024));
    };
    auto emit_rope = [&](const int tile) {
        if (QUANT) {
#pragma unroll
            for (int i = 0; i < RP; ++i)
                *reinterpret_cast<u32x4 *>(pool_b + ropee_off + (tile * KT * PITCH * 2 + i * 8 * PITCH * 2)) = rrope[i];
        } else {
            uint16_t *buf = tile ? tile1 : tile0;
#pragma unroll
            for (int i = 0; i < RP; ++i) {
                const int e = tid + i * NW * 64;
                *reinterpret_cast<u32x4 *>(buf + (e >> 3) * PITCH + DN + 8 * (e & 7)) = rrope[i];
            }
        }
    };
    // What product m = 0..67 of a tile (36 of S^T, then 32 of O^T) carries in its shadow for the following
    // tiles.  A matrix product occupies the pipe for 32 clocks and a wave has one instruction stream: about
    // four other instructions ride under a product for free, each further one costs about five clocks, and a
    // product issued right behind another one wastes its shadow.  So the work is dealt out per product and
    // every product ends with a scheduling barrier, which keeps the compiler from bunching it.  With
    // u = m / 4 and e = m % 4:
    //   m < 2 + DMA_PER_TILE   request m-2 of the tile after the next, its cache row numbers read from the row
    //            table two products earlier: the requests go out under the tile's first products, which carry
    //            nothing else, so that the last of them has nearly a whole tile's time to land (spread over
    //            the tile they were still in flight when the next tile wanted them; all at once the requests
    //            of the four waves queue up at the address unit for several hundred cycles)
    //   e == 0   u odd: piece u/2 of the staged next tile is fetched from the staging ring (u == 1 first
    //            waits for that tile's requests, all but the two just issued: requests complete in order);
    //            u == 15: its rope piece
    //   every e  a quarter of the de-quantisation of half u-2 of the next tile, about three vector
    //            instructions per key of the wave's piece (the last four products carry halves 14 and 15)
    static_assert(DMA_PER_TILE >= 2 && DMA_PER_TILE + 2 <= KSTEPS + 2 * DVB, "one request per product");
    int srow[2];
    // one key's dword at a time: step t = 0 .. 4*PER-1 of a half is quarter t%4 of the dword of key t/4
    uint32_t dq_v = 0, dq_c = 0;
    float dq_a = 0.f, dq_b = 0.f;
    auto emit_step = [&](const int tile, const int h, const int t) {
        const int piece = h / 2, hf = h % 2, q = t / 4, e = t % 4;
        const int i = piece * PER + q;
        if (i >= KPW) return;
        const float sc = psc[piece & 1][q];
        if (e == 0) {
            if (hf == 0) pbias[q] = -128.0f * sc;
            dq_v = praw[piece & 1][q][hf] ^ 0x80808080u;
            dq_a = (float)(dq_v & 0xffu);
            dq_b = (float)((dq_v >> 8) & 0xffu);
        } else if (e == 1) {
            dq_c = pack_bf16x2(__builtin_fmaf(dq_a, sc, pbias[q]), __builtin_fmaf(dq_b, sc, pbias[q]));
            dq_a = (float)((dq_v >> 16) & 0xffu);
        } else if (e == 2) {
            dq_b = (float)(dq_v >> 24);
            dq_a = __builtin_fmaf(dq_a, sc, pbias[q]);
        } else {
            const uint32_t c1 = pack_bf16x2(dq_a, __builtin_fmaf(dq_b, sc, pbias[q]));
            if (hf == 0) {
                plow[q][0] = dq_c, plow[q][1] = c1;
            } else {
                u32x4 v;
                v[0] = plow[q][0], v[1] = plow[q][1], v[2] = dq_c, v[3] = c1;
                *reinterpret_cast<u32x4 *>(pool_b + emit_off + (tile * KT * PITCH * 2 + i * PITCH * 2)) = v;
            }
        }
    };
    auto slot_work = [&](const int m, const int tile, const int slot, const int kt2, const int slot2) {
        const int u = m / 4, e = m % 4;
        if (!QUANT) {
            // bf16 cache: the next tile's rows go straight into the other tile buffer, one request per key of
            // this wave under the tile's first products, the rope pieces through registers
            constexpr int NREQ = KT / NW;
            constexpr int ROPE_LOAD_AT = NREQ > KSTEPS ? NREQ : KSTEPS;     // held in registers for twelve products
            const int kt1 = kt2 - KT;
            uint16_t *buf = tile ? tile1 : tile0;
            if (m < NREQ) {
                const int row = rows_lds[(kt1 - k_begin) + wu * NREQ + m];
                dma16(p.kn + (size_t)row * p.kn_pitch + 16 * l,
                      (uint32_t)(uintptr_t)(lds_byte_t *)buf + (uint32_t)((wu * NREQ + m) * PITCH * 2));
            }
            if (m == ROPE_LOAD_AT) {
#pragma unroll
                for (int i = 0; i < RP; ++i) {
                    const int e2 = tid + i * NW * 64;
                    const int row = rows_lds[(kt1 - k_begin) + (e2 >> 3)];
                    rrope[i] = *reinterpret_cast<const u32x4 *>(p.kr + (size_t)row * p.kr_pitch + 16 * (e2 & 7));
                }
            }
            if (m == ROPE_LOAD_AT + 12) emit_rope(tile);
            return;
        }
        if (m == 4) {
            // the staged next tile has landed: everything but the two requests of products 2 and 3
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(2));
            asm volatile("" ::: "memory");
        }
        if (m >= 2 && m - 2 < DMA_PER_TILE) stage_request(slot2, m - 2, srow[m & 1]);
        if (m < DMA_PER_TILE) srow[m & 1] = stage_row(kt2, m);
        if (e == 0) {
            if (u % 2 == 1 && u / 2 < 8) fetch_piece(u / 2, slot);
            if (u == 15) fetch_rope(slot);
        }
        if (u >= 2 && u < 16) {
#pragma unroll
            for (int j = 0; j < PER; ++j) emit_step(tile, u - 2, e * PER + j);
        }
        if (u == 16) {                      // the last four products carry halves 14 and 15
#pragma unroll
            for (int j = 0; j < 2 * PER; ++j) {
                const int idx = e * 2 * PER + j;
                emit_step(tile, 14 + idx / (4 * PER), idx % (4 * PER));
            }
            if (e == 3) emit_rope(tile);
        }
    };
    // the first tile has nothing to hide behind: its staged bytes are fetched in batches of eight keys,
    // so that the LDS round trips overlap instead of following one another
    auto store_tile = [&](const int tile, const int slot) {
        if (QUANT) {
            fetch_rope(slot);
            constexpr int BATCH = KPW < 8 ? KPW : 8;
#pragma unroll
            for (int i0 = 0; i0 < KPW; i0 += BATCH) {
                u32x2 r[BATCH];
                float sc[BATCH];
#pragma unroll
                for (int i = 0; i < BATCH; ++i) {
                    r[i] = *reinterpret_cast<const u32x2 *>(pool_b + fetch_off + (slot * STG_BYTES + (i0 + i) * DN));
                    sc[i] = *reinterpret_cast<const float *>(pool_b + scale_off + (slot * STG_BYTES + (i0 + i) * 16));
                }
#pragma unroll
                for (int i = 0; i < BATCH; ++i) {
                    const float bias = -128.0f * sc[i];
                    const u32x2 lo = dequant4(r[i][0], sc[i], bias), hi = dequant4(r[i][1], sc[i], bias);
                    const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
                    *reinterpret_cast<u32x4 *>(pool_b + emit_off + (tile * KT * PITCH * 2 + (i0 + i) * PITCH * 2)) = v;
                }
            }
        }
        emit_rope(tile);
    };

    __syncthreads();                       // row table complete
    if (QUANT && n_valid > 0) {
        // the staging ring lies above the Q^T staging: the first two tiles set out before the second
        // Q^T pass is collected
        stage_tile(k_begin, 0);
        stage_tile(k_begin + KT, 1);
        collect_q(1, std::integral_constant<int, 2 * DMA_PER_TILE>{});
    } else {
        collect_q(1, std::integral_constant<int, 0>{});
    }
    __syncthreads();                       // every wave holds its Q^T fragments: the tile buffers are free
    if (n_valid > 0) {
        if (QUANT) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(DMA_PER_TILE));              // the first tile has landed
            asm volatile("" ::: "memory");
        } else {
            issue_loads(k_begin, tile0);
        }
        store_tile(0, 0);
    }
    if (!QUANT) __builtin_amdgcn_s_waitcnt(0x0F70);     // this wave's direct requests into the tile have landed
    __syncthreads();
    // All global loads issued so far (Q^T fragments, first tile) are complete from here on, so that
    // inside the loop the only outstanding vector-memory operations are the gathers of later tiles and
    // the compiler's wait counts do not serialise them with the matrix products.
    if (!QUANT) __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0), expcnt and lgkmcnt unconstrained

    // Scores are scaled inside the exponent (one multiply-add per key).  That wants a positive scale: the
    // sign of a negative one moves into Q^T (exact), and a zero one becomes the smallest normal number,
    // under which every finite score still scales to an exponent that rounds to the same probabilities.
    float sc_log2 = p.scale_log2;
    if (sc_log2 < 0.f) {
        sc_log2 = -sc_log2;
#pragma unroll
        for (int i = 0; i < KSTEPS; ++i) {
            u32x4 v = __builtin_bit_cast(u32x4, qf[i]);
            v ^= 0x80008000u;
            qf[i] = __builtin_bit_cast(bf16x8, v);
        }
    }
    if (sc_log2 == 0.f) sc_log2 = 1.17549435e-38f;

    // One tile.  For the int8 cache the parity of the tile number is a compile-time constant (the loop
    // below runs two tiles per trip), so every LDS address in here is a per-lane base plus an immediate
    // offset.
    auto tile_step = [&](auto parity, auto first_tag, const int kt) __attribute__((always_inline)) {
        const int it = parity;
        constexpr bool FIRST = decltype(first_tag)::value;     // the split's first tile (int8 cache only)
        const uint16_t *cur_tile = (it & 1) ? tile1 : tile0;
        // ---- S^T = K . Q^T, LDS reads running one group of four contraction steps ahead
        f32x16 s;
        {
            const uint16_t *arow = cur_tile + tile_row_of(col) * PITCH + 8 * half;
            // operand reads run four products ahead, in a ring of eight fragments
            bf16x8 fa[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) fa[e] = *reinterpret_cast<const bf16x8 *>(arow + 16 * e);
#pragma unroll
            for (int m = 0; m < KSTEPS; ++m) {
                if (m == 0) s_mfma_first(s, fa[0], qf[0]);
                else s_mfma(s, fa[m & 7], qf[m]);
                __builtin_amdgcn_sched_barrier(0);          // the product leads its slot
                if (m + 4 < KSTEPS) fa[(m + 4) & 7] = *reinterpret_cast<const bf16x8 *>(arow + 16 * (m + 4));
                slot_work(m, (it + 1) & 1, (it + 1) & 1, kt + 2 * KT, it & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        s_chain_done(s);

        // ---- online softmax; lane (head, half) holds keys kt + 8*(r/4) + 4*half + r%4
        float mx = -INFINITY;
        if (kt + KT > k_end) {                  // only the split's last tile can hold keys past k_end
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (kt + tile_row_of(8 * (r >> 2) + 4 * half + (r & 3)) >= k_end) s[r] = -INFINITY;
        }
        // the scale is positive here (its sign went into Q^T), so the largest raw score gives the largest
        // scaled one and the scaling itself is folded into the exponent's multiply-add
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
        {
            float lo, hi;
            both_halves(mx, lo, hi);
            mx = fmaxf(lo, hi) * sc_log2;
        }
        // The reference max follows the true max lazily: probabilities may reach 2^RESCALE_TAU, which
        // fp32 sums and bf16 P hold without loss, and the accumulators are rescaled only on a jump.
        const bool upd = mx > m_run + RESCALE_TAU;          // always true on the first tile (m_run = -inf)
        const float m_new = upd ? mx : m_run;
        const float alpha = upd ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
        const bool rescale = upd && l_run > 0.f;            // nothing accumulated yet: nothing to rescale
        // The exponentials of the first sixteen keys are taken here; those of the other sixteen (needed by
        // the second half of the PV products only) ride in the shadow of the first PV groups.
        float lsum = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            s[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], sc_log2, -m_new));      // v_exp_f32; exp2(-inf) = 0
            lsum += s[r];
        }
        m_run = m_new;
        if (!FIRST && __builtin_expect(__any(rescale), 0)) {     // rare: laid out away from the loop body
            mfma_to_valu_fence();
            AccLoop<0, DVB>::scale(o, alpha);
            valu_to_mfma_fence();
        }
        // P^T of the first sixteen keys is packed here; the exponentials of the other sixteen (needed by the
        // second half of the PV products only), their packing and the row sum are dealt out over the first
        // thirteen PV products
        u32x4 pk0, pk1;
#pragma unroll
        for (int e = 0; e < 4; ++e) pk0[e] = pack_bf16x2(s[2 * e], s[2 * e + 1]);
        auto softmax_slice = [&](const int mp) {
            if (mp < 8) {
                s[8 + mp] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[8 + mp], sc_log2, -m_new));
                lsum += s[8 + mp];
            } else if (mp < 12) {
                pk1[mp - 8] = pack_bf16x2(s[8 + 2 * (mp - 8)], s[8 + 2 * (mp - 8) + 1]);
            } else if (mp == 12) {
                float lo, hi;
                both_halves(lsum, lo, hi);
                lsum = lo + hi;
                l_run = l_run * alpha + lsum;
            }
        };

        // ---- O^T += V^T . P^T: product mp = 16*kk + dvb, V^T reads four products ahead in a ring of eight;
        // each product carries its share of the work for the following tiles (slot_work)
        {
            const uint16_t *vbase = cur_tile + (half + 4 * ((l & 15) >> 2)) * PITCH + 16 * ((l >> 4) & 1) + 4 * (l & 3);
            s16x4 va[8][2];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                va[e][0] = lds_read_tr16(vbase + 32 * e);
                va[e][1] = lds_read_tr16(vbase + 32 * e + 2 * PITCH);
            }
#pragma unroll
            for (int mp = 0; mp < 2 * DVB; ++mp) {
                const s16x8 a = __builtin_shufflevector(va[mp & 7][0], va[mp & 7][1], 0, 1, 2, 3, 4, 5, 6, 7);
                if (FIRST && mp < DVB) acc_mfma_first(o[mp], __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, pk0));
                else acc_mfma(o[mp & 15], __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, mp < DVB ? pk0 : pk1));
                __builtin_amdgcn_sched_barrier(0);          // the product leads its slot
                if (mp + 4 < 2 * DVB) {
                    const int m2 = mp + 4;
                    const uint16_t *a0 = vbase + (16 * (m2 >> 4)) * PITCH + 32 * (m2 & 15);
                    va[m2 & 7][0] = lds_read_tr16(a0);
                    va[m2 & 7][1] = lds_read_tr16(a0 + 2 * PITCH);
                }
                softmax_slice(mp);
                slot_work(KSTEPS + mp, (it + 1) & 1, (it + 1) & 1, kt + 2 * KT, it & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (!QUANT) __builtin_amdgcn_s_waitcnt(0x0F70); // this wave's direct requests into the next tile have landed
        __syncthreads();
    };
    {
        // an odd number of tiles is rounded up: the extra tile holds padding rows only, all of them masked
        if (k_begin < k_end) {
            tile_step(std::integral_constant<int, 0>{}, std::true_type{}, k_begin);
            tile_step(std::integral_constant<int, 1>{}, std::false_type{}, k_begin + KT);
        }
        for (int kt = k_begin + 2 * KT; kt < k_end; kt += 2 * KT) {
            tile_step(std::integral_constant<int, 0>{}, std::false_type{}, kt);
            tile_step(std::integral_constant<int, 1>{}, std::false_type{}, kt + KT);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                 // the padding tiles' requests have landed: the pool is quiet

    // ---- epilogue.  Lane (head, half) holds value channels 32*dvb + 8*(r/4) + 4*half + r%4 of its head;
    // written from there each store instruction would touch 32 rows with 8 bytes each.  Each wave
    // instead transposes 128 channels at a time through its own slice of the (now idle) tile
    // memory, so that 16 lanes write 256 contiguous bytes of one head.
    mfma_to_valu_fence();
    {
        // staging slice of this wave: 32 heads x 128 channels of 16 bits, already scaled by 1/l (a lane's
        // registers all belong to its own head) and converted, in 8-byte chunks of four channels; chunk c
        // of head h is stored at chunk c ^ h: the column-wise writes (32 heads, one chunk) and the
        // row-wise reads (two heads, 16 even or odd chunks each) both touch every bank once.
        uint8_t *stage = reinterpret_cast<uint8_t *>(pool) + w * (32 * 256);
        const int head_base = hg * (32 * NW) + w * 32;
        const size_t prow_base = ((size_t)(t - 8 * p.whole_slots) * nsplit + sp) * p.NQ;    // split rows only
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        // FINAL: bf16 result rows; otherwise fp16 partial of a key split (O / l of the split, merged by
        // the combine kernel with weights l * 2^(m - m_max); O / l is a convex combination of
        // de-quantised V rows, so it stays finite in fp16 as long as |int8 * scale| < 65504).
        // ALL: every head of this wave exists, so the stores need no predicate.  Both are uniform
        // and resolved outside the loops: scalar branches inside them cost more than the work.
        auto drain = [&](auto final_tag, auto all_tag) {
            constexpr bool FINAL = decltype(final_tag)::value;
            constexpr bool ALL = decltype(all_tag)::value;
            const int hsub = l >> 4, j = l & 15;          // on the way out: head 4*e + hsub, channels 8*j .. 8*j+7
            uint16_t *dst0 = FINAL ? p.out + ((size_t)t * p.NQ + head_base + hsub) * DN + 8 * j
                                   : p.part_o + (prow_base + head_base + hsub) * DN + 8 * j;
#pragma unroll
            for (int gq = 0; gq < DVB / 4; ++gq) {
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        // the accumulators leave their registers here and nowhere earlier
                        const f32x16 &acc = o[4 * gq + b4];
                        float r0, r1, r2, r3;
                        asm volatile("v_accvgpr_read_b32 %0, %4\n\tv_accvgpr_read_b32 %1, %5\n\tv_accvgpr_read_b32 %2, %6\n\tv_accvgpr_read_b32 %3, %7"
                                     : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                                     : "a"(acc[4 * q4]), "a"(acc[4 * q4 + 1]), "a"(acc[4 * q4 + 2]), "a"(acc[4 * q4 + 3]));
                        const float v0 = r0 * inv, v1 = r1 * inv, v2 = r2 * inv, v3 = r3 * inv;
                        u32x2 pk;
                        pk[0] = FINAL ? pack_bf16x2(v0, v1) : pack_f16x2(v0, v1);
                        pk[1] = FINAL ? pack_bf16x2(v2, v3) : pack_f16x2(v2, v3);
                        *reinterpret_cast<u32x2 *>(stage + col * 256 + 8 * ((8 * b4 + 2 * q4 + half) ^ col)) = pk;
                    }
                // Eight reads go out before the first store waits for its pair: written as assembly, because
                // the compiler pairs every two reads with a wait of their own (eight exposed LDS latencies
                // per chunk instead of two).
#pragma unroll
                for (int e0 = 0; e0 < 8; e0 += 4) {
                    u32x2 lo[4], hi[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int hl = 4 * (e0 + e) + hsub;
                        const uint32_t a_lo = (uint32_t)(uintptr_t)(lds_byte_t *)(stage + hl * 256 + 8 * ((2 * j) ^ hl));
                        const uint32_t a_hi = (uint32_t)(uintptr_t)(lds_byte_t *)(stage + hl * 256 + 8 * ((2 * j + 1) ^ hl));
                        asm volatile("ds_read_b64 %0, %1" : "=v"(lo[e]) : "v"(a_lo) : "memory");
                        asm volatile("ds_read_b64 %0, %1" : "=v"(hi[e]) : "v"(a_hi) : "memory");
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int hl = 4 * (e0 + e) + hsub;
                        asm volatile("" : "+v"(lo[e]), "+v"(hi[e]));
                        const u32x4 v = {lo[e][0], lo[e][1], hi[e][0], hi[e][1]};
                        if (ALL || head_base + hl < p.NQ)
                            *reinterpret_cast<u32x4 *>(dst0 + (size_t)(4 * (e0 + e)) * DN + 128 * gq) = v;
                    }
                }
            }
        };
        const bool all_heads = head_base + 32 <= p.NQ;
        if (nsplit == 1) {
            if (all_heads) drain(std::true_type{}, std::true_type{});
            else drain(std::true_type{}, std::false_type{});
        } else {
            if (all_heads) drain(std::false_type{}, std::true_type{});
            else drain(std::false_type{}, std::false_type{});
        }
        if (nsplit > 1 && half == 0 && head_ok) {
            p.part_ml[(prow_base + head) * 2] = m_run;
            p.part_ml[(prow_base + head) * 2 + 1] = l_run;
        }
    }
}

// Merges the key splits of one query row: out = sum_s w_s O_s / sum_s w_s with w_s = l_s 2^(m_s - m)
// and O_s the split's normalised fp16 partial (all zeros for an empty split, whose weight is zero).
// One wave per (row, head), a lane per 8 value channels.  The (max, sum) pairs of a (row, head) are the
// same for the whole wave and travel through the scalar cache; the NS 16-byte loads of a lane's partials
// are all requested before the first of them is used.  The kernel moves bytes that were written
// microseconds earlier, and what it costs is launch and latency, not arithmetic: measured, more and
// smaller waves are faster than fewer waves with more loads each (2 or 4 (row, head) pairs per wave:
// 8.2 and 10.2 us against 7.0 at 32 rows x 8 splits).  NS = 2, 4 or 8 splits are in flight at a time:
// the smallest that covers the launch's splits.
template <int NS>
__global__ __launch_bounds__(256) void sfa_combine_kernel(const SfaParams p)
{
    const int lane = threadIdx.x & 63;
    // (row, head) among the split rows, which are rows 8 * whole_slots and up
    const int th = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4 + (threadIdx.x >> 6)));
    const int t_first = 8 * p.whole_slots;
    if (th >= (p.T - t_first) * p.NQ) return;
    const int ts = th / p.NQ, head = th - ts * p.NQ;
    const size_t prow0 = (size_t)ts * p.nsplit * p.NQ + head;      // split s: prow0 + s * NQ
    const f32x2 *ml = reinterpret_cast<const f32x2 *>(p.part_ml);
    f16x8 hv[NS];
    f32x2 v[NS];
#pragma unroll
    for (int e = 0; e < NS; ++e) {
        const size_t prow = prow0 + (size_t)(e < p.nsplit ? e : p.nsplit - 1) * p.NQ;
        v[e] = ml[prow];
        hv[e] = *reinterpret_cast<const f16x8 *>(p.part_o + prow * DN + 8 * lane);
    }
    float m = -INFINITY;
#pragma unroll
    for (int e = 0; e < NS; ++e)
        if (e < p.nsplit && v[e][1] > 0.f) m = fmaxf(m, v[e][0]);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
#pragma unroll
    for (int e = 0; e < NS; ++e) {
        const bool live = e < p.nsplit && v[e][1] > 0.f;
        const float wgt = live ? v[e][1] * __builtin_amdgcn_exp2f(v[e][0] - m) : 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] += wgt * (float)hv[e][c];
        wsum += wgt;
    }
    const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
    u32x4 outv;
#pragma unroll
    for (int e = 0; e < 4; ++e) outv[e] = pack_bf16x2(acc[2 * e] * inv, acc[2 * e + 1] * inv);
    *reinterpret_cast<u32x4 *>(p.out + ((size_t)t_first * p.NQ + th) * DN + 8 * lane) = outv;
}

// The same merge for any number of splits, eight at a time (rows with more than eight key splits).
__global__ __launch_bounds__(256) void sfa_combine_many_kernel(const SfaParams p)
{
    constexpr int NS = 8;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int t_first = 8 * p.whole_slots;                         // the split rows are rows t_first and up
    const size_t total = (size_t)(p.T - t_first) * p.NQ * (DN / 8);
    if (gid >= total) return;
    const int c8 = (int)(gid % (DN / 8));
    const size_t th = gid / (DN / 8);
    const int head = (int)(th % p.NQ);
    const int ts = (int)(th / p.NQ);
    const int t = t_first + ts;
    const size_t prow0 = (size_t)ts * p.nsplit * p.NQ + head;      // split s: prow0 + s * NQ
    const f32x2 *ml = reinterpret_cast<const f32x2 *>(p.part_ml);

    float m = -INFINITY;
    for (int s0 = 0; s0 < p.nsplit; s0 += NS) {
        f32x2 v[NS];
#pragma unroll
        for (int e = 0; e < NS; ++e) v[e] = ml[prow0 + (size_t)(s0 + e < p.nsplit ? s0 + e : p.nsplit - 1) * p.NQ];
#pragma unroll
        for (int e = 0; e < NS; ++e)
            if (v[e][1] > 0.f) m = fmaxf(m, v[e][0]);
    }
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
    for (int s0 = 0; s0 < p.nsplit; s0 += NS) {
        f32x2 v[NS];
        f16x8 hv[NS];
#pragma unroll
        for (int e = 0; e < NS; ++e) {
            const size_t prow = prow0 + (size_t)(s0 + e < p.nsplit ? s0 + e : p.nsplit - 1) * p.NQ;
            v[e] = ml[prow];
            hv[e] = *reinterpret_cast<const f16x8 *>(p.part_o + prow * DN + 8 * c8);
        }
#pragma unroll
        for (int e = 0; e < NS; ++e) {
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

// De-quantises whole cache rows once: out[row][c] = bf16_rne(float(int8) * scale[c / 128]), the values the attention
// kernel forms on the way into LDS.  One wave per row, a lane per eight channels.  For launches that select every
// key many times over (a prefill chunk attends its few thousand keys from thousands of query rows), after which
// the kernel takes its bf16-cache form on these rows: the same bits, without the per-tile conversion.
__global__ __launch_bounds__(256) void sfa_dequant_cache_kernel(const int8_t *kn, const int kn_pitch, const uint8_t *ksc, const int ksc_pitch,
                                                                uint16_t *out, const long long rows)
{
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int l = threadIdx.x & 63;
    const u32x2 raw = *reinterpret_cast<const u32x2 *>(kn + (size_t)row * kn_pitch + 8 * l);
    const float sc = reinterpret_cast<const float *>(ksc + (size_t)row * ksc_pitch)[l >> 4];
    const float bias = -128.0f * sc;
    const u32x2 lo = dequant4(raw[0], sc, bias), hi = dequant4(raw[1], sc, bias);
    const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    *reinterpret_cast<u32x4 *>(out + (size_t)row * DN + 8 * l) = v;
}

}  // namespace

hipError_t sfa_launch(const SfaParams &p, hipStream_t stream)
{
    const int rslots = (p.T + 7) / 8;                      // row slots per XCD
    const unsigned grid = (unsigned)(8 * p.hgroups * (p.whole_slots + (rslots - p.whole_slots) * p.nsplit));
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
    if (p.nsplit > 1 && p.T > 8 * p.whole_slots) {
        const int n_th = (p.T - 8 * p.whole_slots) * p.NQ;
        if (p.nsplit > 8) {
            const size_t total = (size_t)n_th * (DN / 8);
            hipLaunchKernelGGL(sfa_combine_many_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
        } else {
            // one wave per (row, head), four waves per workgroup
            const dim3 cgrid((unsigned)((n_th + 3) / 4));
            if (p.nsplit <= 2) hipLaunchKernelGGL(sfa_combine_kernel<2>, cgrid, dim3(256), 0, stream, p);
            else if (p.nsplit <= 4) hipLaunchKernelGGL(sfa_combine_kernel<4>, cgrid, dim3(256), 0, stream, p);
            else hipLaunchKernelGGL(sfa_combine_kernel<8>, cgrid, dim3(256), 0, stream, p);
        }
        e = hipGetLastError();
    }
    return e;
}

hipError_t sfa_dequant_cache(const int8_t *kn, int kn_pitch, const uint8_t *ksc, int ksc_pitch, uint16_t *out, long long rows,
                             hipStream_t stream)
{
    hipLaunchKernelGGL(sfa_dequant_cache_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, kn, kn_pitch, ksc, ksc_pitch, out, rows);
    return hipGetLastError();
}

}  // namespace pto
