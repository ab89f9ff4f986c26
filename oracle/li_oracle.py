"""CPU oracle for the quantized lightning indexer (score + top-k select).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Restates the torch golden ``lightning_indexer_compute`` of the reference example
(examples/models/deepseek_v32_exp/deepseekv32_lightning_indexer_quant.py:184-269;
operator-side statement examples/models/deepseek_v32_exp/
lightning_indexer_quant_impl.py:138-312) and fixes the two things the golden
leaves to its libraries, so that a bit-exact comparison is meaningful:

1. the order of the 64-term head sum (``torch.bmm`` at :244 leaves it to BLAS):
   here ``acc = 0; for h in 0..63: acc = rn32(acc + rn32(w_scale[h] * x[h]))``;
2. the order among equal scores (``torch.topk`` at :259/:266 leaves it open):
   here candidates are ordered by (score descending, position ascending) and
   ``-0.0 == +0.0``.

Arithmetic per batch ``b`` (``cur_seq = act_seq[b]``), query token ``s``, head
``h``, logical key position ``j`` (physical row ``block_table[b][j // bs] * bs +
j % bs``):

    dot     = sum_d int32(q[s,h,d]) * int32(k[row,d])                 exact (:232)
    x       = fp16_rne(relu(dot) * 2**-11)                            (:233-235)
    w_scale = fp16(q_scale[s,h] * weight[s,h])  when both are fp16    (:222)
            = rn32(float(q_scale) * float(weight))  otherwise
    wq      = head sum in the order stated above, fp32                (:244)
    score   = rn32(wq * float(k_scale[row]))                          (:247)

Select, per query token ``s``: ``eff_seq = cur_seq - (S1 - 1 - s)`` (:254); the
candidates are positions ``0 .. eff_seq-1``; output the first ``selected_count``
in the canonical order, padded with ``-1`` (:258-267).

Pinning (tests/test_oracle_li.py):
* dot -- brute-force Python integers on small inputs (the oracle uses an fp32
  matmul, exact because every partial sum is an integer below 2**24).
* x -- exhaustive comparison over a grid of dot values with a rounding written
  independently with integer arithmetic (round half to even at 11 bits).
* head sum -- Python ``fractions``/struct based emulation of fp32 add and mul on
  tiny inputs; order sensitivity demonstrated by a vector whose sum changes if
  the order changes.
* select -- ``sorted(range(n), key=lambda j: (-score[j], j))`` on engineered
  ties, all-equal rows, +-0.0, eff_seq below / at / above selected_count.
* end to end -- agreement with the scalar C statement in ``oracle_c.c`` and
  set-wise agreement (the reference's own tolerance, 0.5 % per row) with a plain
  torch.bmm/torch.topk evaluation.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

__all__ = [
    "RELU_SCALE",
    "w_scale_of",
    "qk_relu_fp16",
    "head_sum",
    "li_scores",
    "li_scores_fp16_dequant",
    "lightning_indexer_fp16_dequant_ref",
    "canonical_topk",
    "lightning_indexer_ref",
]

RELU_SCALE = 1.0 / 2048.0  # LightningIndexerConfigs.extend_param['scale'] (:47)


def _np(t):
    if isinstance(t, torch.Tensor):
        if t.dtype == torch.bfloat16:
            return t.to(torch.float32).numpy()
        return t.numpy()
    return np.asarray(t)


def w_scale_of(q_scale: torch.Tensor, weight: torch.Tensor) -> np.ndarray:
    """Per-(token, head) factor, fp32 array of q_scale's shape (golden :222)."""
    if q_scale.dtype == torch.float16 and weight.dtype == torch.float16:
        return (q_scale * weight).to(torch.float32).numpy()
    return (q_scale.to(torch.float32) * weight.to(torch.float32)).numpy()


def qk_relu_fp16(q_hd: np.ndarray, k_jd: np.ndarray) -> np.ndarray:
    """x[h, j] = float32(fp16_rne(relu(q_h . k_j) / 2048)) for int8 q [H,D], k [n,D]."""
    dot = q_hd.astype(np.float32) @ k_jd.astype(np.float32).T  # exact: |partial sums| < 2**24
    r = np.maximum(dot, np.float32(0.0)) * np.float32(RELU_SCALE)
    return r.astype(np.float16).astype(np.float32)


def head_sum(w_scale_h: np.ndarray, x_hj: np.ndarray) -> np.ndarray:
    """Sequential fp32 head sum, h ascending, product rounded before the add."""
    acc = np.zeros(x_hj.shape[1], dtype=np.float32)
    w = w_scale_h.astype(np.float32)
    for h in range(x_hj.shape[0]):
        prod = w[h] * x_hj[h]          # fp32 elementwise: one rounding
        acc = acc + prod                 # fp32 elementwise: one rounding
    return acc


def li_scores(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight,
              act_seq_key: Sequence[int], block_table, s1: int | None = None) -> list[np.ndarray]:
    """Score rows.  Returns a list over query tokens t = b*S1+s of fp32 arrays of
    length ``cur_seq[b]`` (logical key order)."""
    q = _np(idx_query)                       # [T, H, D] int8
    t_tot, nh, d = q.shape
    bt = _np(block_table)
    b = len(act_seq_key)
    if s1 is None:
        s1 = t_tot // b
    key = _np(idx_key_cache).reshape(-1, d)  # [NB*bs, D]
    bs = idx_key_cache.shape[1]
    ks = idx_key_scale.reshape(-1).to(torch.float32).numpy()
    w_scale = w_scale_of(idx_query_scale.reshape(t_tot, nh), idx_weight.reshape(t_tot, nh))
    rows = []
    for b_idx in range(b):
        cur = int(act_seq_key[b_idx])
        pos = np.arange(cur, dtype=np.int64)
        phys = bt[b_idx].astype(np.int64)[pos // bs] * bs + pos % bs
        k_sel = key[phys]
        ks_sel = ks[phys]
        for s in range(s1):
            t = b_idx * s1 + s
            x = qk_relu_fp16(q[t], k_sel)
            wq = head_sum(w_scale[t], x)
            rows.append((wq * ks_sel).astype(np.float32))
    return rows


def li_scores_fp16_dequant(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight,
                           act_seq_key: Sequence[int], block_table, s1: int | None = None) -> list[np.ndarray]:
    """Score rows in the arithmetic of the reference's chained C++ operator (golden:
    framework/tests/st/operator/src/test_deepseek_v3.2_exp/gen_lightning_indexer.py:243-257; graph:
    framework/src/operator/models/deepseek_v3.2_exp/lightning_indexer.cpp:183-191), all scales and weights fp16:

        v = fp16(float32(dot) * 2**-11)        signed
        v = fp16(fp16(v * q_scale[h]) * k_scale[j])
        v = max(v, 0);  v = fp16(v * weight[h])
        score[j] = sum_h float32(v)            fp32, h ascending (the golden's torch.sum leaves the order open)

    A product of two fp16 values is exact in fp32, so numpy's float16 multiply (computed in fp32, rounded once) is
    the correctly rounded fp16 product."""
    q = _np(idx_query)
    t_tot, nh, d = q.shape
    bt = _np(block_table)
    b = len(act_seq_key)
    if s1 is None:
        s1 = t_tot // b
    key = _np(idx_key_cache).reshape(-1, d)
    bs = idx_key_cache.shape[1]
    assert idx_query_scale.dtype == idx_key_scale.dtype == idx_weight.dtype == torch.float16
    ks = idx_key_scale.reshape(-1).numpy()
    qs = idx_query_scale.reshape(t_tot, nh).numpy()
    wt = idx_weight.reshape(t_tot, nh).numpy()
    rows = []
    for b_idx in range(b):
        cur = int(act_seq_key[b_idx])
        pos = np.arange(cur, dtype=np.int64)
        phys = bt[b_idx].astype(np.int64)[pos // bs] * bs + pos % bs
        k_sel = key[phys]
        ks_sel = ks[phys]
        for s in range(s1):
            t = b_idx * s1 + s
            dot = q[t].astype(np.float32) @ k_sel.astype(np.float32).T                   # [H, n], exact
            v = (dot * np.float32(RELU_SCALE)).astype(np.float16)
            v = (v * qs[t][:, None]).astype(np.float16)
            v = (v * ks_sel[None, :]).astype(np.float16)
            v = np.maximum(v, np.float16(0.0))
            v = (v * wt[t][:, None]).astype(np.float16)
            acc = np.zeros(cur, dtype=np.float32)
            for h in range(nh):
                acc = acc + v[h].astype(np.float32)
            rows.append(acc)
    return rows


def lightning_indexer_fp16_dequant_ref(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight,
                                       act_seq_key, block_table, selected_count: int = 2048) -> torch.Tensor:
    """Full indexer in the chained operator's arithmetic: topk_res [T, 1, selected_count] int32."""
    t_tot = idx_query.shape[0]
    act = [int(v) for v in (act_seq_key.tolist() if hasattr(act_seq_key, "tolist") else act_seq_key)]
    b = len(act)
    s1 = t_tot // b
    rows = li_scores_fp16_dequant(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act, block_table, s1)
    res = np.empty((t_tot, 1, selected_count), dtype=np.int32)
    for b_idx in range(b):
        for s in range(s1):
            t = b_idx * s1 + s
            res[t, 0] = canonical_topk(rows[t], act[b_idx] - (s1 - 1 - s), selected_count)
    return torch.from_numpy(res)


def canonical_topk(score: np.ndarray, eff_seq: int, k: int) -> np.ndarray:
    """First ``k`` positions of ``0..eff_seq-1`` ordered by (score desc, position
    asc); ``-0.0 == +0.0``; padded with -1.  int32 array of length k."""
    out = np.full(k, -1, dtype=np.int32)
    n = max(min(int(eff_seq), score.shape[0]), 0)
    if n == 0:
        return out
    s = score[:n].astype(np.float32)
    order = np.argsort(-s, kind="stable")    # stable => ascending position among equals
    m = min(n, k)
    out[:m] = order[:m].astype(np.int32)
    return out


def lightning_indexer_ref(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight,
                          act_seq_key, block_table, selected_count: int = 2048) -> torch.Tensor:
    """Full indexer: returns topk_res [T, 1, selected_count] int32."""
    t_tot = idx_query.shape[0]
    act = [int(v) for v in (act_seq_key.tolist() if hasattr(act_seq_key, "tolist") else act_seq_key)]
    b = len(act)
    s1 = t_tot // b
    rows = li_scores(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act, block_table, s1)
    res = np.empty((t_tot, 1, selected_count), dtype=np.int32)
    for b_idx in range(b):
        for s in range(s1):
            t = b_idx * s1 + s
            eff = act[b_idx] - (s1 - 1 - s)
            res[t, 0] = canonical_topk(rows[t], eff, selected_count)
    return torch.from_numpy(res)
