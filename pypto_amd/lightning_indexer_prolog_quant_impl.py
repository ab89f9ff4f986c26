"""Lightning-indexer prolog (quantized) -- drop-in operator entry point.

Same callable, argument names and order as ``lightning_indexer_prolog_quant`` of the reference example
(examples/models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:507-562), and the same four
dataclasses its driver fills (:70-125).  ``configs`` carries NPU tiling hints and is accepted and ignored;
``attrs.eps`` is the layer-norm epsilon, ``attrs.layerout_query`` must be ``"TND"`` and
``attrs.layerout_key`` ``"PA_BSND"`` (the only layouts the reference graph implements, :325-504).

The three weight matrices are taken in plain row-major form -- ``w_qb (q_lora_rank, n_heads*128)`` int8,
``wk (h, 128)`` and ``w_proj (h, n_heads)`` bf16 -- where the reference driver hands over their NPU
fractal re-layout of the same logical matrices (deepseekv32_lightning_indexer_prolog_quant.py:380-386).

Outputs are pre-allocated by the caller and written in place: ``q_int8_out``, ``q_scale_out``,
``weights_out``, and rows ``k_cache_index_in[i]`` of the key cache and its scale array
(``k_int8_out``/``k_scale_out`` normally alias ``k_int8_in``/``k_scale_in``, as in the reference driver
:404-405; when they do not, the cache is copied first).  Returns ``None``; runs asynchronously on the
current stream.

Every fp32 sum has a fixed order and the results are bit-reproducible below 64 tokens.  From 64 tokens on (prefill
chunks) two module attributes choose: by default the query rows' Hadamard sums run on the matrix cores -- the same
exact products added in the cores' order; ``q_int8`` may then differ by one step and ``q_scale`` in its last bit in
rare rows, which the reference's acceptance rule allows for these outputs
(deepseekv32_lightning_indexer_prolog_quant.py:424-425) -- while the key row and the weights, for which that rule
allows no outlier, keep their fixed order.  ``EXACT_SUMS = True`` keeps every sum in its fixed order at any size;
``MATRIX_CORE_HIDDEN_SUMS = True`` also takes the sums over the hidden axis on the matrix cores (``n_heads`` a multiple
of 8), the fastest form: the key row's scale and the weights may then differ by one rounding step of their bf16
intermediate in rare entries.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import _native
from .converter import as_torch, copy_unless_same


@dataclass
class IndexerPrologQuantInput:
    x: torch.Tensor              # bf16 (t, h)
    q_norm: torch.Tensor         # int8 (t, q_lora_rank)
    q_norm_scale: torch.Tensor   # fp32 (t, 1)
    w_qb: torch.Tensor           # int8 (q_lora_rank, head_num * head_dim)
    w_qb_scale: torch.Tensor     # fp32 (head_num * head_dim, 1)
    wk: torch.Tensor             # bf16 (h, head_dim)
    w_proj: torch.Tensor         # bf16 (h, head_num)
    ln_gamma_k: torch.Tensor     # bf16 (head_dim,)
    ln_beta_k: torch.Tensor      # bf16 (head_dim,)
    cos_idx_rope: torch.Tensor   # bf16 (t, rope_head_dim)
    sin_idx_rope: torch.Tensor   # bf16 (t, rope_head_dim)
    hadamard_q: torch.Tensor     # bf16 (head_dim, head_dim)
    hadamard_k: torch.Tensor     # bf16 (head_dim, head_dim)
    k_cache: torch.Tensor        # int8 (block_num, block_size, n_kv, head_dim)
    k_cache_scale: torch.Tensor  # fp16 (block_num, block_size, n_kv, 1)
    k_cache_index: torch.Tensor  # int64 (t,)


@dataclass
class IndexerPrologQuantOutput:
    q_int8: torch.Tensor
    q_scale: torch.Tensor
    k_int8: torch.Tensor
    k_scale: torch.Tensor
    weights: torch.Tensor


@dataclass
class IndexerPrologQuantAttr:
    eps: float = 1e-6
    layerout_query: str = "TND"
    layerout_key: str = "PA_BSND"


@dataclass
class IndexerPrologQuantConfigs:
    q_linear: List[int] = field(default_factory=lambda: [16, 16, 512, 512, 128, 128])
    q_hd: List[int] = field(default_factory=lambda: [32, 32, 128, 128, 128, 128])
    k_linear: List[int] = field(default_factory=lambda: [16, 16, 512, 512, 64, 64])
    w_linear: List[int] = field(default_factory=lambda: [16, 16, 1024, 1024, 32, 32])
    unroll_list: List[int] = field(default_factory=lambda: [32, 16, 8, 4, 2, 1])
    cube_l1_reuse_setting: dict = field(default_factory=lambda: {1: 4})
    mg_copyin_upper_bound: int = 2 * 1024 * 1024
    pg_upper_bound: int = 8192
    block_size: int = 128
    t_sub_tile: int = 1
    chunk_size: int = 2
    vec_nbuffer_mode: int = 0


HEAD_DIM = 128
EXACT_SUMS = False
MATRIX_CORE_HIDDEN_SUMS = False


def _sum_mode() -> int:
    return 1 if EXACT_SUMS else (2 if MATRIX_CORE_HIDDEN_SUMS else 0)
ROPE_DIM = 64


def _need(t: torch.Tensor, name: str, dtype, numel: Optional[int] = None):
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name}: expected {numel} elements, got {t.numel()}")


def lightning_indexer_prolog_quant(x_in, q_norm_in, q_norm_scale_in, w_qb_in, w_qb_scale_in, wk_in, w_proj_in,
                                   ln_gamma_k_in, ln_beta_k_in, cos_idx_rope_in, sin_idx_rope_in, hadamard_q_in,
                                   hadamard_k_in, k_int8_in, k_scale_in, k_cache_index_in, q_int8_out, q_scale_out,
                                   k_int8_out, k_scale_out, weights_out, attrs=None, configs=None, _collect=None):
    C = _native.load()
    attrs = attrs if attrs is not None else IndexerPrologQuantAttr()
    if getattr(attrs, "layerout_query", "TND") != "TND" or getattr(attrs, "layerout_key", "PA_BSND") != "PA_BSND":
        raise ValueError("lightning_indexer_prolog_quant: only layerout_query='TND' and layerout_key='PA_BSND' exist")
    names = ("x_in", "q_norm_in", "q_norm_scale_in", "w_qb_in", "w_qb_scale_in", "wk_in", "w_proj_in", "ln_gamma_k_in",
             "ln_beta_k_in", "cos_idx_rope_in", "sin_idx_rope_in", "hadamard_q_in", "hadamard_k_in", "k_int8_in",
             "k_scale_in", "k_cache_index_in", "q_int8_out", "q_scale_out", "k_int8_out", "k_scale_out", "weights_out")
    vals = (x_in, q_norm_in, q_norm_scale_in, w_qb_in, w_qb_scale_in, wk_in, w_proj_in, ln_gamma_k_in, ln_beta_k_in,
            cos_idx_rope_in, sin_idx_rope_in, hadamard_q_in, hadamard_k_in, k_int8_in, k_scale_in, k_cache_index_in,
            q_int8_out, q_scale_out, k_int8_out, k_scale_out, weights_out)
    (x, qn, qns, wqb, wqbs, wk, wp, gam, bet, cos, sin, hq, hk, kc_in, ks_in, kidx, qo, qso, kc, ks, wo) = \
        [as_torch(v, n) for v, n in zip(vals, names)]

    dev = x.device
    if dev.type != "cuda":
        raise RuntimeError("lightning_indexer_prolog_quant: tensors must live on the GPU (device type 'cuda' on ROCm)")
    if any(t.device != dev for t in (qn, qns, wqb, wqbs, wk, wp, gam, bet, cos, sin, hq, hk, kc_in, ks_in, kidx, qo,
                                     qso, kc, ks, wo)):
        raise RuntimeError("not all tensors are on the same device")
    if x.dim() != 2 or qn.dim() != 2 or wqb.dim() != 2 or wk.dim() != 2 or wp.dim() != 2 or kc.dim() != 4:
        raise ValueError("x, q_norm, w_qb, wk, w_proj must be 2-D (row-major matrices) and the key cache 4-D")
    t, h = x.shape
    q_lora = qn.shape[1]
    n_heads = wp.shape[1]
    if hq.shape != (HEAD_DIM, HEAD_DIM) or hk.shape != (HEAD_DIM, HEAD_DIM):
        raise ValueError(f"hadamard_q/hadamard_k: expected ({HEAD_DIM}, {HEAD_DIM})")
    if cos.shape[-1] != ROPE_DIM or sin.shape[-1] != ROPE_DIM:
        raise ValueError(f"cos_idx_rope/sin_idx_rope: expected rope dimension {ROPE_DIM}")
    if kc.shape[2] != 1 or kc.shape[3] != HEAD_DIM:
        raise ValueError("key cache: expected shape (block_num, block_size, 1, 128)")
    cache_rows = kc.shape[0] * kc.shape[1]
    bf = torch.bfloat16
    _need(x, "x_in", bf)
    _need(qn, "q_norm_in", torch.int8, t * q_lora)
    _need(qns, "q_norm_scale_in", torch.float32, t)
    _need(wqb, "w_qb_in", torch.int8, q_lora * n_heads * HEAD_DIM)
    _need(wqbs, "w_qb_scale_in", torch.float32, n_heads * HEAD_DIM)
    _need(wk, "wk_in", bf, h * HEAD_DIM)
    _need(wp, "w_proj_in", bf, h * n_heads)
    _need(gam, "ln_gamma_k_in", bf, HEAD_DIM)
    _need(bet, "ln_beta_k_in", bf, HEAD_DIM)
    _need(cos, "cos_idx_rope_in", bf, t * ROPE_DIM)
    _need(sin, "sin_idx_rope_in", bf, t * ROPE_DIM)
    _need(hq, "hadamard_q_in", bf)
    _need(hk, "hadamard_k_in", bf)
    _need(kc, "k_int8_out", torch.int8)
    _need(ks, "k_scale_out", torch.float16, cache_rows)
    _need(kidx, "k_cache_index_in", torch.int64, t)
    _need(qo, "q_int8_out", torch.int8, t * n_heads * HEAD_DIM)
    _need(qso, "q_scale_out", torch.float16, t * n_heads)
    _need(wo, "weights_out", torch.float16, t * n_heads)
    if wqb.shape != (q_lora, n_heads * HEAD_DIM) or wk.shape != (h, HEAD_DIM):
        raise ValueError("w_qb must be (q_lora_rank, n_heads*128) and wk (h, 128)")
    if kc_in.shape != kc.shape or ks_in.numel() != ks.numel():
        raise ValueError("k_int8_in/k_scale_in and k_int8_out/k_scale_out differ in shape")
    copy_unless_same(kc, kc_in, "k_int8")
    copy_unless_same(ks, ks_in, "k_scale")

    if _collect is not None:
        # half of the fused operator: checked here, launched by the caller together with the other half
        _collect.append(dict(ptrs=[v.data_ptr() for v in (x, qn, qns, wqb, wqbs, wk, wp, gam, bet, cos, sin, hq, hk, kc, ks, kidx,
                                                          qo, qso, wo)],
                             t=t, h=h, q_lora=q_lora, n_heads=n_heads, cache_rows=cache_rows, eps=float(attrs.eps), sum_mode=_sum_mode()))
        return None
    ws_bytes = C.li_prolog_quant_workspace_bytes(t, h, q_lora, n_heads, cache_rows)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        C.li_prolog_quant_launch(x.data_ptr(), qn.data_ptr(), qns.data_ptr(), wqb.data_ptr(), wqbs.data_ptr(),
                                 wk.data_ptr(), wp.data_ptr(), gam.data_ptr(), bet.data_ptr(), cos.data_ptr(),
                                 sin.data_ptr(), hq.data_ptr(), hk.data_ptr(), kc.data_ptr(), ks.data_ptr(),
                                 kidx.data_ptr(), qo.data_ptr(), qso.data_ptr(), wo.data_ptr(), ws.data_ptr(), ws_bytes,
                                 t, h, q_lora, n_heads, cache_rows, float(attrs.eps), _sum_mode(), stream)
    return None
