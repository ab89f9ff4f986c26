// Launch parameters of the lightning-indexer kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

constexpr int LI_MAX_SELECT = 2048;     // most indices one query token can receive
constexpr int LI_MAX_SEQ = 128 * 1024;  // longest key sequence
constexpr int LI_HEADS = 64;
constexpr int LI_DIM = 128;
constexpr int LI_MAX_BALANCED_TOKENS = 512; // most query tokens the balanced run mapping of the score kernel handles
constexpr int LI_SAMPLE_GROUP = 16;        // the score kernel leaves one sampled score per this many positions
constexpr int LI_MAX_PAIRS_PER_WAVE = 32;  // a wave keeps one cache-row index per 32-key block of its run in a lane

struct LiParams {
    const int8_t *q;        // [T, 64, 128]
    const void *q_scale;    // [T, 64]    q_dt
    const int8_t *kcache;   // [nblocks*bs, 128]
    const void *k_scale;    // [nblocks*bs]  k_dt
    const void *weight;     // [T, 64]    w_dt
    const int32_t *act;     // [B]
    const int32_t *bt;      // [B, maxblk]
    int32_t *topk_res;      // [T, k]
    float *scores;          // workspace [T, score_stride]
    float *sample;          // workspace [T, score_stride / 16]: one score of every 16 consecutive positions
    long long score_stride;
    int T, B, S1, bs, maxblk, nblocks, k;
    int q_dt, k_dt, w_dt;   // PTO_DT_* codes
    int ppw;                // 64-key block pairs per wave of the score kernel, <= LI_MAX_PAIRS_PER_WAVE
    int balanced;           // score kernel sizes its runs from the sequence lengths (units <= LI_MAX_BALANCED_TOKENS)
    int score_wgs;          // its launch size in workgroups of four waves when balanced
    int nt;                 // query tokens of one sequence that a wave of the score kernel scores per key pass: 1 or 2
    int variant;            // 0: fp32 head factors applied after the ReLU; 1: fp16 scales applied before it (all tensors fp16)
};

hipError_t li_launch(const LiParams &p, hipStream_t stream);

}  // namespace pto
