"""MLA prolog (quantized) -- drop-in operator entry points.

Same callables, argument names and order as ``mla_prolog_quant_d`` / ``mla_prolog_quant_p`` of the reference
example (examples/models/deepseek_v32_exp/mla_prolog_quant_impl.py:710-869), with the three configuration
classes its driver fills (:56-94).  ``tile_config`` and ``rope_cfg`` carry NPU tiling hints and are accepted
and ignored.  Built is what these entry points can reach in the reference, the variant of its enabled case
(deepseekv32_mla_prolog_quant.py:790-834): bf16 ``w_dq`` / ``w_dkv_kr``, int8 ``w_uq_qr`` with per-column
``dequant_scale`` (``is_quant_b``), no smoothing.  The reference's ``pre_compute_2d`` also holds branches for int8
down-projections (``is_quant_a``) and a smoothing factor (:413-458, 479-494), but the entry points build their
``MlaQuantInputs()`` themselves and fill in ``dequant_scale_w_uq_qr`` only (:609-614): no argument of
``mla_prolog_quant_d`` / ``_p`` carries the tensors those branches need, and with ``dequant_scale = None`` the
reference fails at ``q_kv[3]`` (:633), so neither has a caller.  ``cache_mode`` is "PA_BSND" or "PA_NZ" as in the
reference, which asserts the value (:591) and does the same for both; anything else raises.  The weight matrices are taken row-major where the reference driver passes their NPU
fractal re-layout (:587-595).  ``k_scale_cache`` is fp32 ``[block_num, block_size, 1, 4]``, the layout the
sparse attention reads.

Outputs are pre-allocated by the caller and written in place: ``q_norm_out``, ``q_norm_scale_out``,
``query_nope_out``, ``query_rope_out`` and rows ``cache_index[i]`` of the three caches (the ``*_out`` cache
arguments normally alias the inputs, as in the reference driver :576-577, 616-617; when they do not, the cache
is copied first).  Returns ``None``; runs asynchronously on the current stream.

``EXACT_ABSORB`` (module attribute, default ``False``) chooses how ``query_nope = query . w_uk`` is summed: on the
matrix cores (the default: the same exact bf16 products, fp32 sums in the cores' order, so some results differ in
the last bf16 bit from the sequential statement -- inside the reference's own acceptance rule for this output,
deepseekv32_mla_prolog_quant.py:668-692) or, when ``True``, as fixed-order fp32 sums that reproduce the
sequential statement bit for bit.  Every other output is the same either way for at most 8 tokens; from 9 tokens
on (larger decode batches, prefill chunks) the default also takes the sums over the hidden axis (``x . w_dq``, ``x . w_dkv_kr``) on the matrix
cores -- sixteen times faster at 512 tokens, the int8 latents then differ by one step in rare entries, inside
the same acceptance rule -- and ``EXACT_ABSORB = True`` keeps every sum in its fixed order.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import _native
from .converter import as_torch, copy_unless_same


EXACT_ABSORB = False


class MlaTileConfig:
    def __init__(self):
        self.tile_b = 8
        self.tile_s = 1
        self.tile_bs = 8
        self.m_tile = 16
        self.mv_tile = 16
        self.pre_quant_cube_tile = [16, 16, 256, 256, 128, 128]
        self.unroll_list = [32, 16, 8, 4, 2, 1]
        self.q_vec_tile0 = 16
        self.q_vec_tile1 = 16
        self.k_vec_tile0 = 16
        self.k_vec_tile1 = 16
        self.cube_l1_reuse_mode = 4
        self.cube_l1_reuse_setting = {}
        self.mg_copyin_upper_bound = 2 * 1024 * 1024
        self.pg_upper_bound = 8192
        self.vec_nbuffer_mode = 1
        self.cube_nbuffer_setting = {3: 4}
        self.dynamic_unaligned_enable = False


@dataclass
class MlaQuantInputs:
    dequant_scale_x: Optional[torch.Tensor] = None
    dequant_scale_w_dq: Optional[torch.Tensor] = None
    dequant_scale_w_uq_qr: Optional[torch.Tensor] = None
    dequant_scale_w_dkv_kr: Optional[torch.Tensor] = None
    quant_scale_ckv: Optional[torch.Tensor] = None
    quant_scale_ckr: Optional[torch.Tensor] = None
    smooth_scales_cq: Optional[torch.Tensor] = None


@dataclass
class RopeTileShapeConfig:
    two_dim: List[int] = field(default_factory=lambda: [128, 128])
    three_dim: List[int] = field(default_factory=lambda: [128, 128, 128])
    four_dim: List[int] = field(default_factory=lambda: [16, 128, 128, 128])


NOPE, ROPE, KV_RANK = 128, 64, 512


def _need(t: torch.Tensor, name: str, dtype, numel: Optional[int] = None):
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name}: expected {numel} elements, got {t.numel()}")


def _mla_prolog_quant(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin, cache_index,
                      kv_cache, kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out, query_rope_out,
                      kv_cache_out, kr_cache_out, k_scale_cache_out, epsilon_cq, epsilon_ckv, cache_mode, tile_config,
                      rope_cfg, _collect=None):
    C = _native.load()
    if cache_mode not in ("PA_BSND", "PA_NZ"):      # the reference asserts the same two and treats them alike (:591)
        raise ValueError(f"mla_prolog_quant: cache_mode must be 'PA_BSND' or 'PA_NZ', got {cache_mode!r}")
    if dequant_scale is None:
        raise ValueError("mla_prolog_quant: dequant_scale is None (the non-quantized w_uq_qr variant is not built)")
    names = ("token_x", "w_dq", "w_uq_qr", "dequant_scale", "w_uk", "w_dkv_kr", "gamma_cq", "gamma_ckv", "cos", "sin",
             "cache_index", "kv_cache", "kr_cache", "k_scale_cache", "q_norm_out", "q_norm_scale_out", "query_nope_out",
             "query_rope_out", "kv_cache_out", "kr_cache_out", "k_scale_cache_out")
    vals = (token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin, cache_index, kv_cache,
            kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out, query_rope_out, kv_cache_out,
            kr_cache_out, k_scale_cache_out)
    (x, wdq, wuq, dqs, wuk, wdkv, gcq, gckv, cs, sn, cidx, kvc_in, krc_in, ksc_in, qn, qns, qnope, qrope, kvc, krc, ksc) = \
        [as_torch(v, n) for v, n in zip(vals, names)]
    dev = x.device
    if dev.type != "cuda":
        raise RuntimeError("mla_prolog_quant: tensors must live on the GPU (device type 'cuda' on ROCm)")
    if any(t.device != dev for t in (wdq, wuq, dqs, wuk, wdkv, gcq, gckv, cs, sn, cidx, kvc_in, krc_in, ksc_in, qn, qns,
                                     qnope, qrope, kvc, krc, ksc)):
        raise RuntimeError("not all tensors are on the same device")
    if x.dim() != 2 or wdq.dim() != 2 or wuq.dim() != 2 or wuk.dim() != 3 or wdkv.dim() != 2 or kvc.dim() != 4:
        raise ValueError("token_x, w_dq, w_uq_qr, w_dkv_kr must be 2-D (row-major matrices), w_uk 3-D, the caches 4-D")
    bf = torch.bfloat16
    if wdq.dtype != bf or wdkv.dtype != bf:
        raise TypeError("mla_prolog_quant: w_dq / w_dkv_kr must be bf16 (the int8 down-projection variant is not built)")
    if wuq.dtype != torch.int8:
        raise TypeError("mla_prolog_quant: w_uq_qr must be int8 (the non-quantized variant is not built)")
    t, h = x.shape
    q_lora = wdq.shape[1]
    n_heads = wuk.shape[0]
    if wuk.shape[1:] != (NOPE, KV_RANK):
        raise ValueError(f"w_uk: expected (n_heads, {NOPE}, {KV_RANK})")
    if wuq.shape != (q_lora, n_heads * (NOPE + ROPE)) or wdkv.shape != (h, KV_RANK + ROPE) or wdq.shape[0] != h:
        raise ValueError("w_dq must be (h, q_lora_rank), w_uq_qr (q_lora_rank, n_heads*192), w_dkv_kr (h, 576)")
    if kvc.shape[2:] != (1, KV_RANK) or krc.shape[2:] != (1, ROPE):
        raise ValueError("caches: expected kv_cache (block_num, block_size, 1, 512) and kr_cache (.., 1, 64)")
    cache_rows = kvc.shape[0] * kvc.shape[1]
    _need(x, "token_x", bf)
    _need(dqs, "dequant_scale", torch.float32, n_heads * (NOPE + ROPE))
    _need(wuk, "w_uk", bf)
    _need(gcq, "gamma_cq", bf, q_lora)
    _need(gckv, "gamma_ckv", bf, KV_RANK)
    _need(cs, "cos", bf, t * ROPE)
    _need(sn, "sin", bf, t * ROPE)
    _need(cidx, "cache_index", torch.int64, t)
    _need(kvc, "kv_cache_out", torch.int8)
    _need(krc, "kr_cache_out", bf, cache_rows * ROPE)
    _need(ksc, "k_scale_cache_out", torch.float32, cache_rows * 4)
    _need(qn, "q_norm_out", torch.int8, t * q_lora)
    _need(qns, "q_norm_scale_out", torch.float32, t)
    _need(qnope, "query_nope_out", bf, t * n_heads * KV_RANK)
    _need(qrope, "query_rope_out", bf, t * n_heads * ROPE)
    for a, b_, nm in ((kvc, kvc_in, "kv_cache"), (krc, krc_in, "kr_cache"), (ksc, ksc_in, "k_scale_cache")):
        if a.numel() != b_.numel() or a.dtype != b_.dtype:
            raise ValueError(f"{nm} and {nm}_out differ in shape or type")
        copy_unless_same(a, b_, nm)

    if _collect is not None:
        # half of the fused operator: checked here, launched by the caller together with the other half
        _collect.append(dict(ptrs=[v.data_ptr() for v in (x, wdq, wuq, dqs, wuk, wdkv, gcq, gckv, cs, sn, cidx, kvc, krc, ksc, qn,
                                                          qns, qnope, qrope)],
                             t=t, h=h, q_lora=q_lora, n_heads=n_heads, cache_rows=cache_rows, eps_cq=float(epsilon_cq),
                             eps_ckv=float(epsilon_ckv), absorb_exact=bool(EXACT_ABSORB), device=dev))
        return None
    ws_bytes = C.mla_prolog_quant_workspace_bytes(t, h, q_lora, n_heads, cache_rows)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        C.mla_prolog_quant_launch(x.data_ptr(), wdq.data_ptr(), wuq.data_ptr(), dqs.data_ptr(), wuk.data_ptr(),
                                  wdkv.data_ptr(), gcq.data_ptr(), gckv.data_ptr(), cs.data_ptr(), sn.data_ptr(),
                                  cidx.data_ptr(), kvc.data_ptr(), krc.data_ptr(), ksc.data_ptr(), qn.data_ptr(),
                                  qns.data_ptr(), qnope.data_ptr(), qrope.data_ptr(), ws.data_ptr(), ws_bytes, t, h,
                                  q_lora, n_heads, cache_rows, float(epsilon_cq), float(epsilon_ckv), bool(EXACT_ABSORB),
                                  stream)
    return None


def mla_prolog_quant_d(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin, cache_index,
                       kv_cache, kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out, query_rope_out,
                       kv_cache_out, kr_cache_out, k_scale_cache_out, epsilon_cq, epsilon_ckv, cache_mode="PA_BSND",
                       tile_config=None, rope_cfg=None, _collect=None):
    """Decode entry point (reference :798-869)."""
    return _mla_prolog_quant(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin,
                             cache_index, kv_cache, kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out,
                             query_rope_out, kv_cache_out, kr_cache_out, k_scale_cache_out, epsilon_cq, epsilon_ckv,
                             cache_mode, tile_config, rope_cfg, _collect)


def mla_prolog_quant_p(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin, cache_index,
                       kv_cache, kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out, query_rope_out,
                       kv_cache_out, kr_cache_out, k_scale_cache_out, epsilon_cq, epsilon_ckv, cache_mode="PA_BSND",
                       tile_config=None, rope_cfg=None, _collect=None):
    """Prefill entry point (reference :717-788); the same kernels."""
    return _mla_prolog_quant(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin,
                             cache_index, kv_cache, kr_cache, k_scale_cache, q_norm_out, q_norm_scale_out, query_nope_out,
                             query_rope_out, kv_cache_out, kr_cache_out, k_scale_cache_out, epsilon_cq, epsilon_ckv,
                             cache_mode, tile_config, rope_cfg, _collect)
