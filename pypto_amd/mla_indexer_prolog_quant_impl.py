"""MLA prolog + lightning-indexer prolog in one call -- drop-in operator entry points.

Same callables, argument names and order as ``mla_indexer_prolog_quant_d`` / ``mla_indexer_prolog_quant_p`` of
the reference example (examples/models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:49-138, 141-256): the
MLA prolog runs first; its int8 normalised query latent and that latent's scale -- intermediates the caller
never sees (:218-219) -- are the indexer prolog's ``q_norm`` / ``q_norm_scale``; hidden states, rope tables and
cache index are shared.  One launch call of the library (``pto_mla_indexer_prolog_quant_launch``: five kernels on the
current stream, the last launches of the two halves merged into one) and one workspace, in which the two
intermediates live; see the two operators'
modules for layouts and for what is built.  Returns ``None``.
"""
from __future__ import annotations

import torch

from . import _native
from .converter import as_torch
from .lightning_indexer_prolog_quant_impl import lightning_indexer_prolog_quant
from .mla_prolog_quant_impl import mla_prolog_quant_d, mla_prolog_quant_p


def _fused(mla_op, token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq, mla_gamma_ckv,
           cos, sin, cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache, ip_w_qb_in, ip_w_qb_scale_in, ip_wk_in,
           ip_w_proj_in, ip_ln_gamma_k_in, ip_ln_beta_k_in, ip_hadamard_q_in, ip_hadamard_k_in, ip_k_cache,
           ip_k_cache_scale, mla_query_nope_out, mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out,
           mla_k_scale_cache_out, ip_q_int8_out, ip_q_scale_out, ip_k_int8_out, ip_k_scale_out, ip_weights_out,
           mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, mla_tile_config, ip_attrs, ip_configs, rope_cfg):
    C = _native.load()
    x = as_torch(token_x, "token_x")
    w_qb = as_torch(ip_w_qb_in, "ip_w_qb_in")
    w_uk = as_torch(mla_w_uk, "mla_w_uk")
    w_proj = as_torch(ip_w_proj_in, "ip_w_proj_in")
    kvc = as_torch(mla_kv_cache_out, "mla_kv_cache_out")
    kc = as_torch(ip_k_int8_out, "ip_k_int8_out")
    if x.dim() != 2 or w_qb.dim() != 2 or w_uk.dim() != 3 or w_proj.dim() != 2 or kvc.dim() != 4 or kc.dim() != 4:
        raise ValueError("token_x, ip_w_qb_in, ip_w_proj_in must be 2-D, mla_w_uk 3-D, the caches 4-D")
    if x.device.type != "cuda":
        raise RuntimeError("mla_indexer_prolog_quant: tensors must live on the GPU (device type 'cuda' on ROCm)")
    t, h = x.shape
    q_lora_rank = w_qb.shape[0]
    # one workspace for the whole operator: the int8 query latent and its scale (the intermediates the caller
    # never sees) in front, then the partial sums of the two halves
    ws_bytes = C.mla_indexer_prolog_quant_workspace_bytes(t, h, q_lora_rank, w_uk.shape[0], kvc.shape[0] * kvc.shape[1],
                                                          w_proj.shape[1], kc.shape[0] * kc.shape[1])
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    qn_bytes = (t * q_lora_rank + 255) // 256 * 256
    q_norm = ws[:t * q_lora_rank].view(torch.int8).view(t, q_lora_rank)
    q_norm_scale = ws[qn_bytes:qn_bytes + 4 * t].view(torch.float32).view(t, 1)
    # each half checks its own arguments exactly as the separate operators do, and hands back raw pointers
    parts = []
    mla_op(token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq, mla_gamma_ckv, cos, sin,
           cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache, q_norm, q_norm_scale, mla_query_nope_out,
           mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out, mla_k_scale_cache_out, mla_epsilon_cq, mla_epsilon_ckv,
           mla_cache_mode, mla_tile_config, rope_cfg, _collect=parts)
    lightning_indexer_prolog_quant(token_x, q_norm, q_norm_scale, ip_w_qb_in, ip_w_qb_scale_in, ip_wk_in, ip_w_proj_in,
                                   ip_ln_gamma_k_in, ip_ln_beta_k_in, cos, sin, ip_hadamard_q_in, ip_hadamard_k_in,
                                   ip_k_cache, ip_k_cache_scale, cache_index, ip_q_int8_out, ip_q_scale_out,
                                   ip_k_int8_out, ip_k_scale_out, ip_weights_out, ip_attrs, ip_configs, _collect=parts)
    m, i = parts
    if (i["t"], i["h"], i["q_lora"]) != (m["t"], m["h"], m["q_lora"]):
        raise ValueError("the two halves disagree about tokens, hidden size or q_lora_rank")
    stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        C.mla_indexer_prolog_quant_launch(m["ptrs"], i["ptrs"], ws.data_ptr(), ws_bytes, m["t"], m["h"], m["q_lora"],
                                          m["n_heads"], m["cache_rows"], m["eps_cq"], m["eps_ckv"], m["absorb_exact"],
                                          i["n_heads"], i["cache_rows"], i["eps"], i["sum_mode"], stream)
    return None


def mla_indexer_prolog_quant_d(*args, **kwargs):
    """Decode entry point (reference :141-256); 41 positional arguments in the reference's order."""
    return _fused(mla_prolog_quant_d, *args, **kwargs)


def mla_indexer_prolog_quant_p(*args, **kwargs):
    """Prefill entry point (reference :49-138); the same kernels."""
    return _fused(mla_prolog_quant_p, *args, **kwargs)
