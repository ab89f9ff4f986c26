// Launch parameters of the sparse-flash-attention kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

constexpr int SFA_MAX_CHUNK = 2048;   // most keys one workgroup handles (row-translation table in LDS)
constexpr int SFA_KEY_TILE = 32;

struct SfaParams {
    const uint16_t *q_nope;   // [T*NQ, 512] bf16
    const uint16_t *q_rope;   // [T*NQ, 64]  bf16
    // The three parts of a cache row, each with its own base and row pitch in bytes: separate arrays
    // (pitches 512 / 128 / 16) or one packed array of 656-byte rows (512 int8 | 64 bf16 | 4 fp32).
    const int8_t *kn;         // 512 int8 latent values
    const uint8_t *kr;        // 64 bf16 rope values
    const uint8_t *ksc;       // 4 fp32 scales, one per 128 latent channels
    int kn_pitch, kr_pitch, ksc_pitch;
    int kn_bf16;              // the latent part is bf16 (1024 bytes, no scales) instead of int8
    const int32_t *topk_idx;  // [T, topk]
    const int32_t *bt;        // [B, maxblk]
    const int32_t *act;       // [B]
    uint16_t *out;            // [T*NQ, 512] bf16
    uint16_t *part_o;         // [split rows, nsplit, NQ, 512] fp16: O / l of each key split (nsplit > 1)
    float *part_ml;           // [split rows, nsplit, NQ, 2]   reference max (log2 domain) and row sum of the split
    long long kv_rows;
    int T, S1, NQ, topk, bs, maxblk;
    int nsplit;               // key splits per query row, of the rows that are split
    int whole_slots;          // rows 0 .. 8 * whole_slots - 1 are not split (one workgroup per row and head group): the
                              // full rounds of a launch of more rows than compute units; 0 = every row is split alike
    int hgroups;              // head groups per query row (32*waves heads each)
    int waves;                // waves per workgroup: 1, 2 or 4
    float scale_log2;         // softmax_scale * log2(e)
};

hipError_t sfa_launch(const SfaParams &p, hipStream_t stream);
// the int8 latent part of `rows` cache rows as bf16 [rows, 512] (what the attention kernel de-quantises them to)
hipError_t sfa_dequant_cache(const int8_t *kn, int kn_pitch, const uint8_t *ksc, int ksc_pitch, uint16_t *out, long long rows,
                             hipStream_t stream);

}  // namespace pto
