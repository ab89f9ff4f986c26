"""CPU oracle for sparse flash attention over the paged int8 latent-KV cache.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Restates, in vectorised torch-CPU form, the torch golden functions of the
reference example (paths relative to the reference tree):

* ``compute_attention_no_flash``  examples/models/deepseek_v32_exp/
  deepseekv32_sparse_flash_attention_quant.py:169-254  -> :func:`sfa_single_pass`
* ``compute_attention`` (online softmax)  same file :49-166 -> :func:`sfa_online`
* page-table arithmetic  same file :215-221 and
  framework/src/interface/tileop/a2a3/dynamic/vector_dyn.h:4197-4204
  -> :func:`page_translate`, :func:`gather_rows`
* int8 de-quantisation  same file :230-234 -> :func:`dequant_kn`

Rounding points kept from the golden: ``bf16_rne(float(int8) * scale)`` for the
latent rows; scores are fp32 sums of exact bf16 products; ``* softmax_scale`` in
fp32; max / exp / sum in fp32; single-pass: ``P = bf16(p / l)`` then fp32 PV then
bf16; online: ``P = bf16(p)`` un-normalised, fp32 PV, rescale by
``exp(m_old - m_new)``, final ``bf16(acc / l)``.

One deliberate difference: the golden never assigns the output of a query row
with ``cur_seq == 0`` (it is left stale); here such rows are defined as zeros.
The golden also only indexes correctly when ``s2_tile == topk`` (it offsets the
already-sliced index row a second time, :207 + :216-217); :func:`sfa_online`
indexes correctly for any tile.

Pinning (tests/test_oracle_sfa.py):
* page_translate / gather_rows -- the reference docstring known-answer
  (python/pypto/experimental.py:64-87) and the ``10*row+col`` buffer recipe of
  python/tests/st/test_gatherinub.py:89-155.
* dequant_kn -- exhaustive over all 256 int8 values against a bit-level bf16
  rounding written independently with integer arithmetic.
* sfa_single_pass / sfa_online -- dense special case against
  ``torch.nn.functional.scaled_dot_product_attention`` in fp64; identical-keys
  invariant; permutation invariance; ``cur_seq`` special cases; cross-check
  against the independent scalar C statement in ``oracle_c.c``.
"""
from __future__ import annotations

import math
from typing import Sequence

import torch

__all__ = [
    "cur_seq_of",
    "page_translate",
    "gather_rows",
    "dequant_kn",
    "sfa_single_pass",
    "sfa_online",
    "sfa_literal_loops",
]


def cur_seq_of(act_seq: int, s1: int, s1_idx: int, topk: int) -> int:
    """Number of selected keys a query row attends to (golden :197)."""
    return min(max(int(act_seq) - s1 + 1 + s1_idx, 0), topk)


def page_translate(logical_idx: torch.Tensor, block_table_row: torch.Tensor, block_size: int) -> torch.Tensor:
    """logical token position -> physical cache row (golden :218-221)."""
    li = logical_idx.to(torch.int64)
    blk = torch.div(li, block_size, rounding_mode="floor")
    return block_table_row.to(torch.int64)[blk] * block_size + li % block_size


def gather_rows(param: torch.Tensor, indices: torch.Tensor, block_table_row: torch.Tensor,
                block_size: int) -> torch.Tensor:
    """``out[j] = param[block_table[idx[j] // bs] * bs + idx[j] % bs]``."""
    return param[page_translate(indices.reshape(-1), block_table_row.reshape(-1), block_size)]


def dequant_kn(kn_rows: torch.Tensor, scale_rows: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """int8 rows [n, 512] x fp32 scales [n, 4] -> ``dtype`` rows (golden :231-234).

    Channel ``c`` uses scale ``c // 128``; the product is an fp32 multiply which is
    then rounded to ``dtype`` (round-to-nearest-even).
    """
    n, dk = kn_rows.shape
    groups = scale_rows.shape[1]
    g = dk // groups
    x = kn_rows.reshape(n * groups, g).to(torch.float32)
    s = scale_rows.to(torch.float32).reshape(n * groups, 1)
    return (x * s).reshape(n, dk).to(dtype)


def _prep(q, topk_indices, topk):
    b, s1, n1, _ = q.shape
    if topk_indices.ndim > 2:
        topk_indices = topk_indices.reshape(b * s1, topk)
    return b, s1, n1, topk_indices


def _selected(b_idx, row, cur_seq, kn, kr, kn_scales, topk_indices, block_table, block_size, is_kn_quant, dtype):
    idx = topk_indices[row, :cur_seq]
    phys = page_translate(idx, block_table[b_idx], block_size)
    if is_kn_quant:
        kn_sel = dequant_kn(kn[phys], kn_scales[phys], dtype)
    else:
        kn_sel = kn[phys]
    return kn_sel, kr[phys]


def sfa_single_pass(q, kn, kr, kn_scales, topk_indices, block_table, actual_seq: Sequence[int],
                    block_size: int, scalar: float, topk: int, is_kn_quant: bool = True) -> torch.Tensor:
    """The golden the reference compares against (single softmax pass).

    q [B,S1,N,Dn+Dr] bf16 (nope ‖ rope); kn [rows,Dn] int8 (or bf16); kr [rows,Dr]
    bf16; kn_scales [rows,4] fp32; topk_indices [B*S1, topk] int32;
    block_table [B, MB] int32; returns [B,S1,N,Dn] in q's dtype.
    """
    b, s1, n1, topk_indices = _prep(q, topk_indices, topk)
    dn = kn.shape[1]
    dtype = q.dtype
    out = torch.zeros([b, s1, n1, dn], dtype=dtype)
    for b_idx in range(b):
        for s1_idx in range(s1):
            cur = cur_seq_of(actual_seq[b_idx], s1, s1_idx, topk)
            if cur == 0:
                continue
            kn_sel, kr_sel = _selected(b_idx, b_idx * s1 + s1_idx, cur, kn, kr, kn_scales, topk_indices,
                                       block_table, block_size, is_kn_quant, dtype)
            kj = torch.cat([kn_sel, kr_sel], dim=-1).to(torch.float32)
            sij = torch.matmul(q[b_idx, s1_idx].to(torch.float32), kj.t())
            sij = sij * scalar
            m = sij.amax(dim=-1, keepdim=True)
            p = torch.exp(sij - m)
            l = p.sum(dim=-1, keepdim=True)
            pn = (p / l).to(dtype)
            o = torch.matmul(pn.to(torch.float32), kn_sel.to(torch.float32))
            out[b_idx, s1_idx] = o.to(dtype)
    return out


def sfa_online(q, kn, kr, kn_scales, topk_indices, block_table, actual_seq: Sequence[int],
               block_size: int, scalar: float, topk: int, s2_tile: int, is_kn_quant: bool = True) -> torch.Tensor:
    """Online-softmax golden (golden :49-166) with correct indexing for any tile."""
    b, s1, n1, topk_indices = _prep(q, topk_indices, topk)
    dn = kn.shape[1]
    dtype = q.dtype
    out = torch.zeros([b, s1, n1, dn], dtype=dtype)
    for b_idx in range(b):
        for s1_idx in range(s1):
            cur = cur_seq_of(actual_seq[b_idx], s1, s1_idx, topk)
            if cur == 0:
                continue
            kn_all, kr_all = _selected(b_idx, b_idx * s1 + s1_idx, cur, kn, kr, kn_scales, topk_indices,
                                       block_table, block_size, is_kn_quant, dtype)
            qi = q[b_idx, s1_idx].to(torch.float32)
            ntile = math.ceil(cur / s2_tile)
            oi = li = mi = None
            for t in range(ntile):
                lo, hi = t * s2_tile, min((t + 1) * s2_tile, cur)
                kn_t = kn_all[lo:hi]
                kj = torch.cat([kn_t, kr_all[lo:hi]], dim=-1).to(torch.float32)
                sij = torch.matmul(qi, kj.t()) * scalar
                m_t = sij.amax(dim=-1, keepdim=True)
                p = torch.exp(sij - m_t)
                q1 = torch.matmul(p.to(dtype).to(torch.float32), kn_t.to(torch.float32))
                l_t = p.sum(dim=-1, keepdim=True)
                if t == 0:
                    oi, li, mi = q1, l_t, m_t
                else:
                    m_new = torch.maximum(mi, m_t)
                    a_old = torch.exp(mi - m_new)
                    a_new = torch.exp(m_t - m_new)
                    li = a_old * li + a_new * l_t
                    oi = oi * a_old + q1 * a_new
                    mi = m_new
            out[b_idx, s1_idx] = (oi / li).to(dtype)
    return out


def sfa_literal_loops(q, kn, kr, kn_scales, topk_indices, block_table, actual_seq, block_size, scalar, topk):
    """Per-element loop form (one Python iteration per selected key), the shape of
    the golden's gather at :215-228.  Only for tiny cases and for timing the cost
    of that formulation."""
    b, s1, n1, topk_indices = _prep(q, topk_indices, topk)
    dn, dr = kn.shape[1], kr.shape[1]
    dtype = q.dtype
    out = torch.zeros([b, s1, n1, dn], dtype=dtype)
    for b_idx in range(b):
        for s1_idx in range(s1):
            cur = cur_seq_of(actual_seq[b_idx], s1, s1_idx, topk)
            if cur == 0:
                continue
            row = topk_indices[b_idx * s1 + s1_idx]
            slc_kn = torch.zeros([cur, dn], dtype=kn.dtype)
            slc_kr = torch.zeros([cur, dr], dtype=dtype)
            slc_sc = torch.zeros([cur, 4], dtype=torch.float32)
            for j in range(cur):
                t = int(row[j])
                phys = int(block_table[b_idx, t // block_size]) * block_size + t % block_size
                slc_kn[j] = kn[phys]
                slc_kr[j] = kr[phys]
                slc_sc[j] = kn_scales[phys]
            kn_t = (slc_kn.reshape(-1, 128).to(torch.float32) * slc_sc.reshape(-1, 1)).reshape(-1, dn).to(dtype)
            kj = torch.cat([kn_t, slc_kr], dim=-1)
            sij = torch.matmul(q[b_idx, s1_idx].to(torch.float32), kj.t().to(torch.float32)) * scalar
            m = sij.amax(dim=-1, keepdim=True)
            p = torch.exp(sij - m)
            l = p.sum(dim=-1, keepdim=True)
            o = torch.matmul((p / l).to(dtype).to(torch.float32), kn_t.to(torch.float32))
            out[b_idx, s1_idx] = o.to(dtype)
    return out


def unpack_nope_cache(nope_cache_2d: torch.Tensor):
    """``[rows, 656] int8`` -> (kn [rows,512] int8, kr [rows,64] bf16, scales [rows,4] fp32): the byte
    ranges the packed-cache golden reads (deepseekv32_sparse_attention_antiquant.py:109-118:
    ``[:, :512]`` int8, ``[:, 512:640]`` viewed as the activation dtype, ``[:, 640:]`` viewed as fp32)."""
    rows = nope_cache_2d.shape[0]
    kn = nope_cache_2d[:, :512].contiguous()
    kr = nope_cache_2d[:, 512:640].contiguous().view(torch.bfloat16).reshape(rows, 64)
    sc = nope_cache_2d[:, 640:656].contiguous().view(torch.float32).reshape(rows, 4)
    return kn, kr, sc


def sa_antiquant_single_pass(q, nope_cache_2d, topk_indices, block_table, actual_seq: Sequence[int],
                             block_size: int, scalar: float, topk: int) -> torch.Tensor:
    """Golden of the packed-cache operator, compute_attention_aq
    (deepseekv32_sparse_attention_antiquant.py:49-136): gather whole 656-byte rows, split them, then
    exactly the arithmetic of the three-array golden (dequant :109-118, scores :121, softmax :124-130,
    PV :133).  The reference runs it with s2_tile == topk (:283), where its tile loop is one pass."""
    kn, kr, sc = unpack_nope_cache(nope_cache_2d)
    return sfa_single_pass(q, kn, kr, sc, topk_indices, block_table, actual_seq, block_size, scalar, topk)
