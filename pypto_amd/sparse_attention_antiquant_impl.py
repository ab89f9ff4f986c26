"""Sparse attention over the packed quantized cache -- drop-in operator entry points.

Same module name, callables, argument names and order as the reference example
examples/models/deepseek_v32_exp/sparse_attention_antiquant_impl.py: ``SaTileShapeConfig`` (:35-42),
``sparse_attention_antiquant_d`` (:263-300) and ``sparse_attention_antiquant_p`` (:322-359).  The
computation is that of ``sparse_flash_attention_quant_d``; only the cache layout differs: one array
``nope_cache [block_num*block_size, 656] int8`` whose rows hold 512 int8 latent values, the 64 bf16
rope values (bytes 512..639) and the 4 fp32 scales (bytes 640..655), as packed by the reference
driver (deepseekv32_sparse_attention_antiquant.py:258-268).  One row is one contiguous 656-byte read.

Calling convention as for the other operators: ``from_torch`` wrappers or bare torch tensors, output
pre-allocated and written in place, ``None`` returned, asynchronous on the current stream;
``tile_config`` is accepted and ignored.
"""
from __future__ import annotations

import torch

from . import _native
from .converter import as_torch
from .sparse_flash_attention_quant_impl import KV_LORA_RANK, ROPE_DIM, SaTileShapeConfig, _check  # noqa: F401

PACKED_ROW_BYTES = KV_LORA_RANK + 2 * ROPE_DIM + 4 * 4     # 656


def _launch(query_nope, query_rope, nope_cache, topk_indices, block_table, kv_act_seqs, attention_out, nq, n_kv,
            softmax_scale, topk, block_size, max_blocknum_perbatch, num_splits=0):
    C = _native.load()
    qn = as_torch(query_nope, "query_nope")
    qr = as_torch(query_rope, "query_rope")
    nc = as_torch(nope_cache, "nope_cache")
    ti = as_torch(topk_indices, "topk_indices")
    bt = as_torch(block_table, "block_table")
    act = as_torch(kv_act_seqs, "kv_act_seqs")
    out = as_torch(attention_out, "attention_out")

    tensors = (qn, qr, nc, ti, bt, act, out)
    dev = qn.device
    if dev.type != "cuda":
        raise RuntimeError("sparse_attention_antiquant: tensors must live on the GPU (device type 'cuda' on ROCm)")
    if any(t.device != dev for t in tensors):
        raise RuntimeError("not all tensors are on the same device")   # python/pypto/runtime.py:224-228

    _check(qn, "query_nope", torch.bfloat16, 2)
    _check(qr, "query_rope", torch.bfloat16, 2)
    _check(nc, "nope_cache", torch.int8, 2)
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
    rows = nc.shape[0]
    if nc.shape[1] != PACKED_ROW_BYTES:
        raise ValueError(f"nope_cache: expected [rows, {PACKED_ROW_BYTES}], got {tuple(nc.shape)}")
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
        C.sa_antiquant_launch(qn.data_ptr(), qr.data_ptr(), nc.data_ptr(), ti.data_ptr(), bt.data_ptr(), act.data_ptr(),
                              out.data_ptr(), ws.data_ptr(), ws_bytes, b, s1, nq, n_kv, topk, block_size, bt_cols, rows,
                              float(softmax_scale), int(num_splits), stream)
    return None


def sparse_attention_antiquant_d(query_nope, query_rope, nope_cache, topk_indices,
                                 block_table, kv_act_seqs, attention_out,
                                 nq, n_kv, softmax_scale, topk, block_size,
                                 max_blocknum_perbatch, tile_config=None):
    """Decode entry point.  Arguments as in the reference (:263-294):

    query_nope (t*n_q, 512) bf16; query_rope (t*n_q, 64) bf16; nope_cache (block_num*block_size, 656) int8;
    topk_indices (t, n_kv*topk) int32; block_table (b, max_blocknum_perbatch) int32; kv_act_seqs (b,) int32;
    attention_out (b, s, n_q, 512) bf16, written in place.
    """
    return _launch(query_nope, query_rope, nope_cache, topk_indices, block_table, kv_act_seqs, attention_out, nq, n_kv,
                   softmax_scale, topk, block_size, max_blocknum_perbatch)


def sparse_attention_antiquant_p(query_nope, query_rope, nope_cache, topk_indices,
                                 block_table, kv_act_seqs, attention_out,
                                 nq, n_kv, softmax_scale, topk, block_size,
                                 max_blocknum_perbatch, tile_config=None):
    """Prefill entry point (:322-359); same computation and arguments as the decode one."""
    return _launch(query_nope, query_rope, nope_cache, topk_indices, block_table, kv_act_seqs, attention_out, nq, n_kv,
                   softmax_scale, topk, block_size, max_blocknum_perbatch)
