"""Sparse flash attention (quantized latent KV) -- drop-in operator entry points.

Same module name, callables, argument names and order as the reference example
examples/models/deepseek_v32_exp/sparse_flash_attention_quant_impl.py:
``SaTileShapeConfig`` (:35-42), ``sparse_flash_attention_quant_d`` (:437-476) and
``sparse_flash_attention_quant_p`` (:499-538).  As in the reference's legacy jit convention
(python/pypto/runtime.py:218-253) tensors are handed over with ``from_torch`` (bare torch tensors
are accepted too), the output tensor is pre-allocated by the caller and written in place, the call
returns ``None`` and runs asynchronously on the current stream.

What changes underneath: instead of tracing a tile graph and compiling it for an NPU, the call
validates the arguments and launches the hand-written gfx950 kernels through the C ABI
(include/pypto_amd_sfa.h).  ``tile_config`` carries NPU tiling hints and is accepted and ignored.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _native
from .converter import as_torch

KV_LORA_RANK = 512
ROPE_DIM = 64


@dataclass
class SaTileShapeConfig:
    g_tile: int
    s_kv_tile: int
    c1_tile_shape: list
    v1_tile_shape: list
    c2_tile_shape: list
    v2_tile_shape: list


def _check(t: torch.Tensor, name: str, dtype, ndim: int):
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name}: expected {ndim} dimensions, got shape {tuple(t.shape)}")


def _launch(query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices, block_table, kv_act_seqs,
            attention_out, nq, n_kv, softmax_scale, topk, block_size, max_blocknum_perbatch, num_splits=0):
    C = _native.load()
    qn = as_torch(query_nope, "query_nope")
    qr = as_torch(query_rope, "query_rope")
    kn = as_torch(key_nope_2d, "key_nope_2d")
    kr = as_torch(key_rope_2d, "key_rope_2d")
    quant = kn.dtype == torch.int8                       # else the non-quantized branch (:149-153, :199-202)
    ks = as_torch(k_nope_scales, "k_nope_scales") if quant or k_nope_scales is not None else None
    ti = as_torch(topk_indices, "topk_indices")
    bt = as_torch(block_table, "block_table")
    act = as_torch(kv_act_seqs, "kv_act_seqs")
    out = as_torch(attention_out, "attention_out")

    tensors = tuple(x for x in (qn, qr, kn, kr, ks, ti, bt, act, out) if x is not None)
    dev = qn.device
    if dev.type != "cuda":
        raise RuntimeError("sparse_flash_attention_quant: tensors must live on the GPU (device type 'cuda' on ROCm)")
    if any(t.device != dev for t in tensors):
        raise RuntimeError("not all tensors are on the same device")   # python/pypto/runtime.py:224-228

    if kn.dtype not in (torch.int8, torch.bfloat16):
        raise TypeError(f"key_nope_2d: expected int8 (quantized cache) or bfloat16, got {kn.dtype}")
    _check(qn, "query_nope", torch.bfloat16, 2)
    _check(qr, "query_rope", torch.bfloat16, 2)
    _check(kn, "key_nope_2d", kn.dtype, 2)
    _check(kr, "key_rope_2d", torch.bfloat16, 2)
    if quant:
        _check(ks, "k_nope_scales", torch.float32, 2)
    _check(ti, "topk_indices", torch.int32, 2)
    _check(bt, "block_table", torch.int32, 2)
    _check(act, "kv_act_seqs", torch.int32, 1)
    _check(out, "attention_out", torch.bfloat16, 4)

    nq, n_kv, topk, block_size = int(nq), int(n_kv), int(topk), int(block_size)
    max_blocknum_perbatch = int(max_blocknum_perbatch)
    b = act.shape[0]
    if qn.shape[1] != KV_LORA_RANK or qr.shape[1] != ROPE_DIM:
        raise ValueError(f"query_nope/query_rope: expected widths {KV_LORA_RANK}/{ROPE_DIM}")
    if qn.shape[0] != qr.shape[0] or qn.shape[0] % (b * nq) != 0:
        raise ValueError("query_nope/query_rope: first dimension must be b*s1*nq")
    s1 = qn.shape[0] // (b * nq)
    rows = kn.shape[0]
    if kn.shape[1] != KV_LORA_RANK or tuple(kr.shape) != (rows, ROPE_DIM) or (quant and tuple(ks.shape) != (rows, 4)):
        raise ValueError("key_nope_2d/key_rope_2d/k_nope_scales: expected [rows,512], [rows,64], [rows,4]")
    if tuple(ti.shape) != (b * s1, n_kv * topk):
        raise ValueError(f"topk_indices: expected shape {(b * s1, n_kv * topk)}, got {tuple(ti.shape)}")
    if bt.shape[0] != b or bt.shape[1] < max_blocknum_perbatch:
        raise ValueError("block_table: expected shape [b, >= max_blocknum_perbatch]")
    if tuple(out.shape) != (b, s1, nq, KV_LORA_RANK):
        raise ValueError(f"attention_out: expected shape {(b, s1, nq, KV_LORA_RANK)}, got {tuple(out.shape)}")

    bt_cols = bt.shape[1]
    ws_bytes = C.sfa_quant_workspace_bytes(b, s1, nq, n_kv, topk, block_size, bt_cols, rows, float(softmax_scale),
                                           int(num_splits))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)   # caching allocator, stream-ordered
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        if quant:
            C.sfa_quant_launch(qn.data_ptr(), qr.data_ptr(), kn.data_ptr(), kr.data_ptr(), ks.data_ptr(), ti.data_ptr(),
                               bt.data_ptr(), act.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, b, s1, nq, n_kv,
                               topk, block_size, bt_cols, rows, float(softmax_scale), int(num_splits), stream)
        else:
            C.sfa_bf16kv_launch(qn.data_ptr(), qr.data_ptr(), kn.data_ptr(), kr.data_ptr(), ti.data_ptr(), bt.data_ptr(),
                                act.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, b, s1, nq, n_kv, topk,
                                block_size, bt_cols, rows, float(softmax_scale), int(num_splits), stream)
    return None


def sparse_flash_attention_quant_d(query_nope, query_rope, key_nope_2d, key_rope_2d,
                                   k_nope_scales, topk_indices, block_table, kv_act_seqs,
                                   attention_out, nq, n_kv, softmax_scale, topk,
                                   block_size, max_blocknum_perbatch, tile_config=None):
    """Decode entry point.  Arguments as in the reference (:437-470):

    query_nope (t*n_q, 512) bf16; query_rope (t*n_q, 64) bf16; key_nope_2d (block_num*block_size, 512)
    int8; key_rope_2d (block_num*block_size, 64) bf16; k_nope_scales (block_num*block_size, 4) fp32;
    topk_indices (t, n_kv*topk) int32; block_table (b, max_blocknum_perbatch) int32; kv_act_seqs (b,)
    int32; attention_out (b, s, n_q, 512) bf16, written in place.
    """
    return _launch(query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices, block_table,
                   kv_act_seqs, attention_out, nq, n_kv, softmax_scale, topk, block_size, max_blocknum_perbatch)


def sparse_flash_attention_quant_p(query_nope, query_rope, key_nope_2d, key_rope_2d,
                                   k_nope_scales, topk_indices, block_table, kv_act_seqs,
                                   attention_out, nq, n_kv, softmax_scale, topk,
                                   block_size, max_blocknum_perbatch, tile_config=None):
    """Prefill entry point (:499-538); same computation and arguments as the decode one."""
    return _launch(query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices, block_table,
                   kv_act_seqs, attention_out, nq, n_kv, softmax_scale, topk, block_size, max_blocknum_perbatch)
