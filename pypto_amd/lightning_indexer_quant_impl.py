"""Lightning indexer (quantized, decode) -- drop-in operator entry point.

Same callable, argument names and order as ``lightning_indexer_decode`` of the reference example
(examples/models/deepseek_v32_exp/lightning_indexer_quant_impl.py:315-346); ``LightningIndexerConfigs``
mirrors the driver's dataclass (deepseekv32_lightning_indexer_quant.py:24-47).  ``unroll_list`` and
``configs`` carry NPU tiling hints and are accepted and ignored -- except that the ReLU scale
``1/2048`` in ``configs.extend_param`` is part of the arithmetic and is what the kernel implements.
The output ``topk_res`` is pre-allocated by the caller and written in place; the call returns
``None`` and runs asynchronously on the current stream.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from . import _native
from .converter import as_torch

MAX_LI_S1 = 4              # reference :30
MAX_LI_S2 = 128 * 1024     # reference :31


@dataclass
class LightningIndexerConfigs:
    mg_copy_in_upper_bound: int = 2 * 1024 * 1024
    pg_upper_bound: int = 16 * 8192
    cube_l1_reuse_setting: dict = field(default_factory=lambda: {0: 16})
    vec_merge_mode: int = 2
    vec_nbuffer_setting: dict = field(default_factory=lambda: {-1: 16})
    s1_tile: int = 2
    topk_tile: int = 16384
    c1_tile: list = field(default_factory=lambda: [64, 64, 128, 128, 128, 128])
    c2_tile: list = field(default_factory=lambda: [128, 128, 64, 64, 128, 128])
    extend_param: dict = field(default_factory=lambda: {"scale": 1 / 2048.0, "relu_type": "RELU"})


_DT = {torch.float16: 0, torch.float32: 1, torch.bfloat16: 2}


def lightning_indexer_decode(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight,
                             act_seq_key, block_table, topk_res, unroll_list=None, configs=None,
                             selected_count: int = 2048, arith_variant: str = "scaled_sum"):
    """idx_query (t, 64, 128) int8; idx_query_scale (t, 64) fp16|fp32; idx_key_cache
    (block_num, block_size, 1, 128) int8; idx_key_scale (block_num, block_size, 1) fp16|fp32;
    idx_weight (t, 64) fp16|bf16|fp32; act_seq_key (b,) int32; block_table (b, max_blocks) int32;
    topk_res (t, 1, selected_count) int32, written in place.

    ``arith_variant`` (not part of the reference signature): ``"scaled_sum"`` is the arithmetic of this
    operator's reference graph and golden; ``"fp16_dequant"`` is that of the reference's chained C++ operator
    (framework/src/operator/models/deepseek_v3.2_exp/lightning_indexer.cpp:149-197; golden
    framework/tests/st/operator/src/test_deepseek_v3.2_exp/gen_lightning_indexer.py:243-257): fp16(q.k/2048) times
    q_scale, times k_scale (both products rounded to fp16), ReLU, times weight in fp16, fp32 head sum.  It takes
    fp16 scales and weights only."""
    C = _native.load()
    q = as_torch(idx_query, "idx_query")
    qs = as_torch(idx_query_scale, "idx_query_scale")
    kc = as_torch(idx_key_cache, "idx_key_cache")
    ks = as_torch(idx_key_scale, "idx_key_scale")
    w = as_torch(idx_weight, "idx_weight")
    act = as_torch(act_seq_key, "act_seq_key")
    bt = as_torch(block_table, "block_table")
    res = as_torch(topk_res, "topk_res")

    dev = q.device
    if dev.type != "cuda":
        raise RuntimeError("lightning_indexer_decode: tensors must live on the GPU (device type 'cuda' on ROCm)")
    if any(t.device != dev for t in (qs, kc, ks, w, act, bt, res)):
        raise RuntimeError("not all tensors are on the same device")
    if q.dtype != torch.int8 or kc.dtype != torch.int8:
        raise TypeError("idx_query/idx_key_cache: expected int8")
    for name, t in (("idx_query_scale", qs), ("idx_key_scale", ks), ("idx_weight", w)):
        if t.dtype not in _DT:
            raise TypeError(f"{name}: expected fp16, fp32 or bf16, got {t.dtype}")
    if act.dtype != torch.int32 or bt.dtype != torch.int32 or res.dtype != torch.int32:
        raise TypeError("act_seq_key/block_table/topk_res: expected int32")
    if q.dim() != 3 or kc.dim() != 4 or bt.dim() != 2 or act.dim() != 1:
        raise ValueError("idx_query must be 3-D, idx_key_cache 4-D, block_table 2-D, act_seq_key 1-D")
    t_tot, n_heads, d = q.shape
    b = act.shape[0]
    block_num, block_size, n_kv, dk = kc.shape
    selected_count = int(selected_count)
    if n_kv != 1 or dk != d:
        raise ValueError("idx_key_cache: expected shape (block_num, block_size, 1, head_dim)")
    if t_tot % b != 0:
        raise ValueError("idx_query: first dimension must be b*s1")
    if t_tot // b > MAX_LI_S1:
        raise ValueError(f"s1 = {t_tot // b} exceeds MAX_LI_S1 = {MAX_LI_S1}")
    if qs.numel() != t_tot * n_heads or w.numel() != t_tot * n_heads:
        raise ValueError("idx_query_scale/idx_weight: expected t*n_heads elements")
    if ks.numel() != block_num * block_size:
        raise ValueError("idx_key_scale: expected block_num*block_size elements")
    if bt.shape[0] != b:
        raise ValueError("block_table: expected first dimension b")
    if res.numel() != t_tot * selected_count:
        raise ValueError(f"topk_res: expected {t_tot}*{selected_count} elements")
    if bt.shape[1] * block_size > MAX_LI_S2:
        raise ValueError(f"block_table spans more than MAX_LI_S2 = {MAX_LI_S2} positions")

    if arith_variant not in ("scaled_sum", "fp16_dequant"):
        raise ValueError(f"arith_variant: expected 'scaled_sum' or 'fp16_dequant', got {arith_variant!r}")
    if arith_variant == "fp16_dequant" and not (qs.dtype == ks.dtype == w.dtype == torch.float16):
        raise TypeError("arith_variant 'fp16_dequant' takes fp16 idx_query_scale, idx_key_scale and idx_weight")
    for name, tt in (("idx_query_scale", qs), ("idx_key_scale", ks), ("idx_weight", w)):
        if not tt.is_contiguous():
            raise ValueError(f"{name}: must be contiguous")
    args = (t_tot, b, n_heads, d, block_num, block_size, bt.shape[1], selected_count, _DT[qs.dtype], _DT[ks.dtype],
            _DT[w.dtype])
    ws_bytes = C.li_decode_workspace_bytes(*args)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        C.li_decode_launch(q.data_ptr(), qs.data_ptr(), kc.data_ptr(), ks.data_ptr(), w.data_ptr(), act.data_ptr(),
                           bt.data_ptr(), res.data_ptr(), ws.data_ptr(), ws_bytes, *args, stream,
                           1 if arith_variant == "fp16_dequant" else 0)
    return None
