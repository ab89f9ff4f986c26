"""MLA prolog + lightning-indexer prolog in one call -- drop-in operator entry points.

Same callables, argument names and order as ``mla_indexer_prolog_quant_d`` / ``mla_indexer_prolog_quant_p`` of
the reference example (examples/models/deepseek_v32_exp/mla_indexer_prolog_quant_impl.py:49-138, 141-256): the
MLA prolog runs first; its int8 normalised query latent and that latent's scale -- intermediates the caller
never sees (:218-219) -- are the indexer prolog's ``q_norm`` / ``q_norm_scale``; hidden states, rope tables and
cache index are shared.  Both stages run back to back on the current stream; see the two operators' modules
for layouts and for what is built.  Returns ``None``.
"""
from __future__ import annotations

import torch

from .converter import as_torch
from .lightning_indexer_prolog_quant_impl import lightning_indexer_prolog_quant
from .mla_prolog_quant_impl import mla_prolog_quant_d, mla_prolog_quant_p


def _fused(mla_op, token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq, mla_gamma_ckv,
           cos, sin, cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache, ip_w_qb_in, ip_w_qb_scale_in, ip_wk_in,
           ip_w_proj_in, ip_ln_gamma_k_in, ip_ln_beta_k_in, ip_hadamard_q_in, ip_hadamard_k_in, ip_k_cache,
           ip_k_cache_scale, mla_query_nope_out, mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out,
           mla_k_scale_cache_out, ip_q_int8_out, ip_q_scale_out, ip_k_int8_out, ip_k_scale_out, ip_weights_out,
           mla_epsilon_cq, mla_epsilon_ckv, mla_cache_mode, mla_tile_config, ip_attrs, ip_configs, rope_cfg):
    x = as_torch(token_x, "token_x")
    w_qb = as_torch(ip_w_qb_in, "ip_w_qb_in")
    t, q_lora_rank = x.shape[0], w_qb.shape[0]
    q_norm = torch.empty([t, q_lora_rank], dtype=torch.int8, device=x.device)
    q_norm_scale = torch.empty([t, 1], dtype=torch.float32, device=x.device)
    mla_op(token_x, mla_w_dq, mla_w_uq_qr, mla_dequant_scale, mla_w_uk, mla_w_dkv_kr, mla_gamma_cq, mla_gamma_ckv, cos, sin,
           cache_index, mla_kv_cache, mla_kr_cache, mla_k_scale_cache, q_norm, q_norm_scale, mla_query_nope_out,
           mla_query_rope_out, mla_kv_cache_out, mla_kr_cache_out, mla_k_scale_cache_out, mla_epsilon_cq, mla_epsilon_ckv,
           mla_cache_mode, mla_tile_config, rope_cfg)
    lightning_indexer_prolog_quant(token_x, q_norm, q_norm_scale, ip_w_qb_in, ip_w_qb_scale_in, ip_wk_in, ip_w_proj_in,
                                   ip_ln_gamma_k_in, ip_ln_beta_k_in, cos, sin, ip_hadamard_q_in, ip_hadamard_k_in,
                                   ip_k_cache, ip_k_cache_scale, cache_index, ip_q_int8_out, ip_q_scale_out,
                                   ip_k_int8_out, ip_k_scale_out, ip_weights_out, ip_attrs, ip_configs)
    return None


def mla_indexer_prolog_quant_d(*args, **kwargs):
    """Decode entry point (reference :141-256); 41 positional arguments in the reference's order."""
    return _fused(mla_prolog_quant_d, *args, **kwargs)


def mla_indexer_prolog_quant_p(*args, **kwargs):
    """Prefill entry point (reference :49-138); the same kernels."""
    return _fused(mla_prolog_quant_p, *args, **kwargs)
